// Mamba-1 selective scan, full sequence.
//
//   h[b,d,n] <- exp(delta[b,t,d] * a_neg[d,n]) * h[b,d,n] + delta*u * B[b,t,n]
//   y[b,t,d]  = sum_n h[b,d,n] * C[b,t,n] + D[d] * u[b,t,d]      (optionally * gate)
//
// Replaces the reference's ssm_parallel_scan_fwd_nosave_* and
// ssm_burnin_forward_nosave_* (kernels/mamba_ssm_parallel.cu:544-765,
// kernels/mamba_ssm.cu:304-400).  Layout is the reference's: activations
// [batch, T, d_inner] with the channel fastest, so 64 consecutive channels sit
// on the 64 lanes of a wave and every activation access is one coalesced row
// segment; the state h[n] of a channel lives in that lane's registers for the
// whole sequence and is written back once.
#include "common.hpp"

namespace mrs {

constexpr int kNPL = 16;  // state entries held per lane

// ---------------------------------------------------------------------------
// Generic sequential kernel.  LPC lanes share one channel, lane g of the group
// owning states n in [16g, 16g+16); any d_state <= 16*LPC, any d_inner.
// One wave per (batch row, tile of 64/LPC channels); time runs serially.
// ---------------------------------------------------------------------------
template <typename T, int LPC, bool S4D, int GATE>
__global__ __launch_bounds__(kWave) void ssm_scan_seq_kernel(
    float *__restrict__ h, T *__restrict__ y, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, const T *__restrict__ Cm, int64_t bc_stride,
    const float *__restrict__ a_neg, const float *__restrict__ Dp, const T *__restrict__ gate,
    int Tlen, int di, int ds, int tiles) {
    constexpr int CPW = kWave / LPC;
    const int b = blockIdx.x / tiles;
    const int tile = blockIdx.x - b * tiles;
    const int lane = threadIdx.x;
    const int g = lane % LPC;
    const int d = tile * CPW + lane / LPC;
    const bool live = d < di;
    const int dd = live ? d : di - 1;  // clamp: dead lanes compute on a valid channel, never store
    const int n0 = g * kNPL;

    float hs[kNPL], a2[kNPL];
#pragma unroll
    for (int j = 0; j < kNPL; j++) {
        const int n = n0 + j;
        const bool nv = n < ds;
        hs[j] = nv ? h[((int64_t)b * di + dd) * ds + n] : 0.0f;
        a2[j] = nv ? a_neg[(int64_t)dd * ds + n] * kLog2e : 0.0f;
    }
    const float a20 = a_neg[(int64_t)dd * ds] * kLog2e;  // S4D: a2[n] = (n+1)*a20
    const float Dd = Dp[dd];

    const int64_t row0 = (int64_t)b * Tlen;
    for (int t = 0; t < Tlen; t++) {
        const int64_t row = row0 + t;
        const int64_t i = row * di + dd;
        const float dl = Store<T>::ld(delta + i);
        const float uu = Store<T>::ld(u + i);
        const float du = dl * uu;
        float acc = (g == 0) ? Dd * uu : 0.0f;
        const T *Br = Bm + row * bc_stride + n0;
        const T *Cr = Cm + row * bc_stride + n0;
        float pw = 0.0f, p1 = 0.0f;
        if (S4D) {
            p1 = fast_exp2(dl * a20);
            pw = (LPC == 1) ? p1 : fast_exp2(dl * a20 * (float)(n0 + 1));
        }
#pragma unroll
        for (int j = 0; j < kNPL; j++) {
            const bool nv = (n0 + j) < ds;
            const float Bn = nv ? Store<T>::ld(Br + j) : 0.0f;
            const float Cn = nv ? Store<T>::ld(Cr + j) : 0.0f;
            float da;
            if (S4D) { da = pw; pw *= p1; }
            else da = fast_exp2(dl * a2[j]);
            hs[j] = fmaf(da, hs[j], du * Bn);
            acc = fmaf(hs[j], Cn, acc);
        }
#pragma unroll
        for (int m = 1; m < LPC; m <<= 1) acc += __shfl_xor(acc, m, kWave);
        if (GATE == 1) acc *= Store<T>::ld(gate + i);
        if (GATE == 2) acc *= silu(Store<T>::ld(gate + i));
        if (live && g == 0) Store<T>::st(y + i, acc);
    }
    if (live) {
#pragma unroll
        for (int j = 0; j < kNPL; j++)
            if (n0 + j < ds) h[((int64_t)b * di + d) * ds + n0 + j] = hs[j];
    }
}

template <typename T, int LPC, bool S4D>
static int launch_seq_gate(hipStream_t st, int gate_mode, float *h, T *y, const T *delta, const T *u,
                           const T *Bm, const T *Cm, int64_t bc_stride, const float *a_neg,
                           const float *D, const T *gate, int batch, int Tlen, int di, int ds) {
    constexpr int CPW = kWave / LPC;
    const int tiles = (di + CPW - 1) / CPW;
    const dim3 grid((unsigned)(batch * tiles)), block(kWave);
#define MRS_LAUNCH(G)                                                                              \
    hipLaunchKernelGGL((ssm_scan_seq_kernel<T, LPC, S4D, G>), grid, block, 0, st, h, y, delta, u, Bm, \
                       Cm, bc_stride, a_neg, D, gate, Tlen, di, ds, tiles)
    if (gate_mode == 0) MRS_LAUNCH(0);
    else if (gate_mode == 1) MRS_LAUNCH(1);
    else MRS_LAUNCH(2);
#undef MRS_LAUNCH
    return check_launch("ssm_scan_seq_kernel");
}

template <typename T>
static int launch_seq(hipStream_t st, bool s4d, int gate_mode, float *h, void *y, const void *delta,
                      const void *u, const void *Bm, const void *Cm, int64_t bc_stride,
                      const float *a_neg, const float *D, const void *gate, int batch, int Tlen,
                      int di, int ds) {
#define MRS_ARGS                                                                                     \
    st, gate_mode, h, (T *)y, (const T *)delta, (const T *)u, (const T *)Bm, (const T *)Cm, bc_stride, \
        a_neg, D, (const T *)gate, batch, Tlen, di, ds
#define MRS_LPC(L) return s4d ? launch_seq_gate<T, L, true>(MRS_ARGS) : launch_seq_gate<T, L, false>(MRS_ARGS)
    if (ds <= 16) { MRS_LPC(1); }
    if (ds <= 32) { MRS_LPC(2); }
    if (ds <= 64) { MRS_LPC(4); }
    if (ds <= 128) { MRS_LPC(8); }
    MRS_LPC(16);
#undef MRS_LPC
#undef MRS_ARGS
}

// ---------------------------------------------------------------------------
// T-split route (d_state == 16).  The sequence is cut into C chunks of L steps;
// one wave owns (batch row, 64-channel tile, chunk), lane = channel, the 16
// states of a channel in that lane's registers, B_t/C_t rows in scalar registers.
//   pass A  chunk_state_kernel: chunk-end state S_c reached from a zero entering
//           state (chunk 0: from the caller's h) and sum_t delta over the chunk,
//           for chunks 0..C-2; also saves a copy of the caller's h.
//   pass B  chunk_out_kernel: folds the summaries of the chunks before it into its
//           entering state  h_in(c) = exp(a * sum delta_{c-1}) h_in(c-1) + S_{c-1},
//           then runs the recurrence over its chunk writing y; the last chunk
//           writes the final state back to h.
// The composition law (a,b)o(a',b') = (aa', a'b + b') makes this equal to the
// serial scan up to rounding.
// ---------------------------------------------------------------------------
struct SplitPlan {
    int nchunk;  // C
    int len;     // L
};

static SplitPlan make_split_plan(int batch, int Tlen, int di) {
    const int tiles = (di + kWave - 1) / kWave;
    const int64_t base = (int64_t)batch * tiles;
    int c = (int)((6144 + base - 1) / base);  // ~6 waves per SIMD on 1024 SIMDs
    if (c > 32) c = 32;                        // the entering-state fold is O(C) per wave
    if (c > Tlen / 32) c = Tlen / 32;          // chunks of at least 32 steps
    if (c < 1) c = 1;
    int len = (Tlen + c - 1) / c;
    len = (len + 3) & ~3;
    c = (Tlen + len - 1) / len;
    return {c, len};
}

static size_t split_workspace_floats(int batch, int di, int nchunk) {
    // h0 copy [B][16][di] + S [B][C-1][16][di] + sum delta [B][C-1][di]
    return (size_t)batch * 16 * di + (size_t)batch * (nchunk - 1) * 17 * di;
}

// One row of B or C (16 values) as uniform f32.  16-bit rows are read as 8 packed
// dwords with scalar loads (the address is wave-uniform), so they cost no VALU/LDS.
template <typename T> struct Row16;
template <> struct Row16<float> {
    __device__ static __forceinline__ void ld(const float *r, float (&o)[16]) {
#pragma unroll
        for (int j = 0; j < 16; j++) o[j] = r[j];
    }
};
template <> struct Row16<bf16_t> {
    __device__ static __forceinline__ void ld(const bf16_t *r, float (&o)[16]) {
        const uint32_t *w = reinterpret_cast<const uint32_t *>(r);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t v = w[j];
            o[2 * j] = __uint_as_float(v << 16);
            o[2 * j + 1] = __uint_as_float(v & 0xffff0000u);
        }
    }
};
template <> struct Row16<f16_t> {
    __device__ static __forceinline__ void ld(const f16_t *r, float (&o)[16]) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 *w = reinterpret_cast<const h2 *>(r);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const h2 v = w[j];
            o[2 * j] = (float)v.x;
            o[2 * j + 1] = (float)v.y;
        }
    }
};

// Decay factors of one step: da[n] = 2^(dl * a2[n]); S4D: a2[n] = (n+1) a2[0] -> powers of one exp.
template <bool S4D>
__device__ __forceinline__ void decay16(float dl, const float (&a2)[16], float (&da)[16]) {
    if (S4D) {
        const float p1 = fast_exp2(dl * a2[0]);
        da[0] = p1;
#pragma unroll
        for (int j = 1; j < 16; j++) da[j] = da[j - 1] * p1;
    } else {
#pragma unroll
        for (int j = 0; j < 16; j++) da[j] = fast_exp2(dl * a2[j]);
    }
}

// Entering state of chunk c from the summaries of chunks 0..c-1 (c >= 1).
template <bool S4D>
__device__ __forceinline__ void fold_entering_state(float (&hs)[16], const float (&a2)[16],
                                                    const float *__restrict__ S, const float *__restrict__ sumd,
                                                    int b, int c, int nchunk, int di, int dd) {
    const int64_t sbase = (int64_t)b * (nchunk - 1);
#pragma unroll
    for (int j = 0; j < 16; j++) hs[j] = S[(sbase * 16 + j) * di + dd];  // S_0 already includes h0
    for (int k = 1; k < c; k++) {
        const float sd = sumd[(sbase + k) * di + dd];
        float da[16];
        decay16<S4D>(sd, a2, da);
#pragma unroll
        for (int j = 0; j < 16; j++) hs[j] = fmaf(da[j], hs[j], S[((sbase + k) * 16 + j) * di + dd]);
    }
}

template <typename T, bool S4D>
__global__ __launch_bounds__(kWave) void chunk_state_kernel(
    const float *__restrict__ h, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, int64_t bc_stride, const float *__restrict__ a_neg,
    float *__restrict__ h0copy, float *__restrict__ S, float *__restrict__ sumd,
    int Tlen, int di, int tiles, int nchunk, int len) {
    const int nc1 = nchunk - 1;
    const int tile = blockIdx.x % tiles;
    const int rest = blockIdx.x / tiles;
    const int c = rest % nc1;
    const int b = rest / nc1;
    const int d = tile * kWave + threadIdx.x;
    const bool live = d < di;
    const int dd = live ? d : di - 1;

    float hs[16], a2[16];
#pragma unroll
    for (int j = 0; j < 16; j++) {
        a2[j] = a_neg[(int64_t)dd * 16 + j] * kLog2e;
        hs[j] = 0.0f;
    }
    if (S4D) {
#pragma unroll
        for (int j = 1; j < 16; j++) a2[j] = a2[0] * (float)(j + 1);
    }
    if (c == 0) {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            hs[j] = h[((int64_t)b * di + dd) * 16 + j];
            if (live) h0copy[((int64_t)b * 16 + j) * di + d] = hs[j];
        }
    }
    const int t0 = c * len, t1 = min(Tlen, t0 + len);
    float sd = 0.0f;
    const int64_t row0 = (int64_t)b * Tlen;
#pragma unroll 2
    for (int t = t0; t < t1; t++) {
        const int64_t row = row0 + t;
        const float dl = Store<T>::ld(delta + row * di + dd);
        const float uu = Store<T>::ld(u + row * di + dd);
        const float du = dl * uu;
        float Bv[16], da[16];
        Row16<T>::ld(Bm + row * bc_stride, Bv);
        decay16<S4D>(dl, a2, da);
        sd += dl;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            hs[j] *= da[j];
            hs[j] = fmaf(du, Bv[j], hs[j]);
        }
    }
    if (live) {
        const int64_t sbase = (int64_t)b * nc1 + c;
#pragma unroll
        for (int j = 0; j < 16; j++) S[(sbase * 16 + j) * di + d] = hs[j];
        sumd[sbase * di + d] = sd;
    }
}

template <typename T, bool S4D, int GATE>
__global__ __launch_bounds__(kWave) void chunk_out_kernel(
    float *__restrict__ h, T *__restrict__ y, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, const T *__restrict__ Cm, int64_t bc_stride,
    const float *__restrict__ a_neg, const float *__restrict__ Dp, const T *__restrict__ gate,
    const float *__restrict__ h0copy, const float *__restrict__ S, const float *__restrict__ sumd,
    int Tlen, int di, int tiles, int nchunk, int len) {
    const int tile = blockIdx.x % tiles;
    const int rest = blockIdx.x / tiles;
    const int c = rest % nchunk;
    const int b = rest / nchunk;
    const int d = tile * kWave + threadIdx.x;
    const bool live = d < di;
    const int dd = live ? d : di - 1;

    float hs[16], a2[16];
#pragma unroll
    for (int j = 0; j < 16; j++) a2[j] = a_neg[(int64_t)dd * 16 + j] * kLog2e;
    if (S4D) {
#pragma unroll
        for (int j = 1; j < 16; j++) a2[j] = a2[0] * (float)(j + 1);
    }
    if (c == 0) {
#pragma unroll
        for (int j = 0; j < 16; j++) hs[j] = h0copy[((int64_t)b * 16 + j) * di + dd];
    } else {
        fold_entering_state<S4D>(hs, a2, S, sumd, b, c, nchunk, di, dd);
    }
    const float Dd = Dp[dd];
    const int t0 = c * len, t1 = min(Tlen, t0 + len);
    const int64_t row0 = (int64_t)b * Tlen;
#pragma unroll 2
    for (int t = t0; t < t1; t++) {
        const int64_t row = row0 + t;
        const int64_t i = row * di + dd;
        const float dl = Store<T>::ld(delta + i);
        const float uu = Store<T>::ld(u + i);
        float g = 1.0f;
        if (GATE) g = Store<T>::ld(gate + i);
        const float du = dl * uu;
        float Bv[16], Cv[16], da[16];
        Row16<T>::ld(Bm + row * bc_stride, Bv);
        Row16<T>::ld(Cm + row * bc_stride, Cv);
        decay16<S4D>(dl, a2, da);
        float acc = Dd * uu;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            hs[j] *= da[j];
            hs[j] = fmaf(du, Bv[j], hs[j]);
            acc = fmaf(hs[j], Cv[j], acc);
        }
        if (GATE == 1) acc *= g;
        if (GATE == 2) acc *= silu(g);
        if (live) Store<T>::st(y + i, acc);
    }
    if (c == nchunk - 1 && live) {
#pragma unroll
        for (int j = 0; j < 16; j++) h[((int64_t)b * di + d) * 16 + j] = hs[j];
    }
}

template <typename T, bool S4D>
static int launch_split_s4d(hipStream_t st, int gate_mode, float *h, T *y, const T *delta, const T *u,
                            const T *Bm, const T *Cm, int64_t bc_stride, const float *a_neg,
                            const float *D, const T *gate, float *ws, SplitPlan plan, int batch,
                            int Tlen, int di) {
    const int tiles = (di + kWave - 1) / kWave;
    const int C = plan.nchunk, L = plan.len;
    float *h0copy = ws;
    float *S = h0copy + (size_t)batch * 16 * di;
    float *sumd = S + (size_t)batch * (C - 1) * 16 * di;
    const dim3 block(kWave);
    const dim3 gridA((unsigned)(batch * (C - 1) * tiles)), gridB((unsigned)(batch * C * tiles));
    hipLaunchKernelGGL((chunk_state_kernel<T, S4D>), gridA, block, 0, st, h, delta, u, Bm, bc_stride, a_neg,
                       h0copy, S, sumd, Tlen, di, tiles, C, L);
    int rc = check_launch("chunk_state_kernel");
    if (rc) return rc;
#define MRS_LAUNCH(G)                                                                                   \
    hipLaunchKernelGGL((chunk_out_kernel<T, S4D, G>), gridB, block, 0, st, h, y, delta, u, Bm, Cm,      \
                       bc_stride, a_neg, D, gate, h0copy, S, sumd, Tlen, di, tiles, C, L)
    if (gate_mode == 0) MRS_LAUNCH(0);
    else if (gate_mode == 1) MRS_LAUNCH(1);
    else MRS_LAUNCH(2);
#undef MRS_LAUNCH
    return check_launch("chunk_out_kernel");
}

template <typename T>
static int launch_split(hipStream_t st, bool s4d, int gate_mode, float *h, void *y, const void *delta,
                        const void *u, const void *Bm, const void *Cm, int64_t bc_stride,
                        const float *a_neg, const float *D, const void *gate, float *ws, SplitPlan plan,
                        int batch, int Tlen, int di) {
#define MRS_ARGS                                                                                       \
    st, gate_mode, h, (T *)y, (const T *)delta, (const T *)u, (const T *)Bm, (const T *)Cm, bc_stride, \
        a_neg, D, (const T *)gate, ws, plan, batch, Tlen, di
    return s4d ? launch_split_s4d<T, true>(MRS_ARGS) : launch_split_s4d<T, false>(MRS_ARGS);
#undef MRS_ARGS
}

static int scan_check(const char *fn, int dtype, const void *h, const void *y, const void *delta,
                      const void *u, const void *B, const void *C, const void *a_neg, const void *D,
                      int64_t bc_stride, int batch, int T, int di, int ds) {
    if (dtype != MRS_F32 && dtype != MRS_F16 && dtype != MRS_BF16)
        return fail(MRS_E_DTYPE, "%s: dtype %d is not f32/f16/bf16", fn, dtype);
    if (!h || !y || !delta || !u || !B || !C || !a_neg || !D) return fail(MRS_E_NULL, "%s: null pointer", fn);
    if (batch < 1 || T < 1 || di < 1) return fail(MRS_E_SHAPE, "%s: batch=%d T=%d d_inner=%d must be >= 1", fn, batch, T, di);
    if (ds < 1 || ds > 256) return fail(MRS_E_SHAPE, "%s: d_state=%d outside 1..=256", fn, ds);
    if (bc_stride < ds) return fail(MRS_E_SHAPE, "%s: bc_stride=%lld < d_state=%d", fn, (long long)bc_stride, ds);
    // reference guard: element counts must fit i32 (src/mamba_ssm/gpu/launch.rs:20-47)
    const int64_t lim = 0x7fffffffLL;
    if ((int64_t)batch * ((int64_t)T + 1) * di * ds > lim)
        return fail(MRS_E_SHAPE, "%s: batch*(T+1)*d_inner*d_state exceeds i32", fn);
    return MRS_OK;
}

}  // namespace mrs

using namespace mrs;

extern "C" size_t mrs_ssm_scan_workspace_bytes(int batch, int T, int d_inner, int d_state) {
    if (batch < 1 || T < 1 || d_inner < 1 || d_state != 16) return 256;
    const SplitPlan plan = make_split_plan(batch, T, d_inner);
    if (plan.nchunk < 2) return 256;
    const size_t bytes = split_workspace_floats(batch, d_inner, plan.nchunk) * sizeof(float);
    return (bytes + 255) & ~(size_t)255;
}

extern "C" int mrs_ssm_scan_fwd_ex(void *stream, int dtype, float *h, void *y, const void *delta,
                                   const void *u, const void *B, const void *C, int64_t bc_stride,
                                   const float *a_neg, const float *D, const void *gate, unsigned flags,
                                   void *workspace, size_t workspace_bytes, int batch, int T,
                                   int d_inner, int d_state) {
    int rc = scan_check("mrs_ssm_scan_fwd_ex", dtype, h, y, delta, u, B, C, a_neg, D, bc_stride, batch, T, d_inner, d_state);
    if (rc) return rc;
    int gate_mode = 0;
    if ((flags & MRS_GATE_PREACT) && (flags & MRS_GATE_SILU))
        return fail(MRS_E_SHAPE, "mrs_ssm_scan_fwd_ex: MRS_GATE_PREACT and MRS_GATE_SILU are exclusive");
    if (flags & MRS_GATE_PREACT) gate_mode = 1;
    if (flags & MRS_GATE_SILU) gate_mode = 2;
    if (gate_mode && !gate) return fail(MRS_E_NULL, "mrs_ssm_scan_fwd_ex: gate flag set but gate is NULL");
    const bool s4d = (flags & MRS_A_S4D_REAL) != 0;
    hipStream_t st = as_stream(stream);
    if ((flags & MRS_FORCE_SEQUENTIAL) && (flags & MRS_FORCE_PARALLEL))
        return fail(MRS_E_SHAPE, "mrs_ssm_scan_fwd_ex: MRS_FORCE_SEQUENTIAL and MRS_FORCE_PARALLEL are exclusive");
    // T-split route: d_state 16, rows of B/C readable as packed dwords, a workspace to put the chunk summaries in.
    const size_t es = (dtype == MRS_F32) ? 4 : 2;
    const bool rows_ok = aligned(B, 4) && aligned(C, 4) && (bc_stride * es) % 4 == 0;
    bool split = d_state == 16 && rows_ok && workspace && !(flags & MRS_FORCE_SEQUENTIAL);
    SplitPlan plan = {1, T};
    if (split) {
        plan = make_split_plan(batch, T, d_inner);
        // the reference's Auto threshold (src/config.rs:21-37): parallel above 256 steps
        if (plan.nchunk < 2 || (T <= 256 && !(flags & MRS_FORCE_PARALLEL))) split = false;
    }
    if ((flags & MRS_FORCE_PARALLEL) && !split && d_state == 16 && T >= 64)
        return fail(MRS_E_WORKSPACE, "mrs_ssm_scan_fwd_ex: MRS_FORCE_PARALLEL needs a workspace and 4-byte aligned B/C rows");
    if (split) {
        const size_t need = split_workspace_floats(batch, d_inner, plan.nchunk) * sizeof(float);
        if (workspace_bytes < need)
            return fail(MRS_E_WORKSPACE, "mrs_ssm_scan_fwd_ex: workspace %zu bytes < %zu needed", workspace_bytes, need);
        if (!aligned(workspace, 256)) return fail(MRS_E_ALIGN, "mrs_ssm_scan_fwd_ex: workspace must be 256-byte aligned");
        MRS_DISPATCH_DTYPE(dtype, T_, return launch_split<T_>(st, s4d, gate_mode, h, y, delta, u, B, C, bc_stride, a_neg, D, gate,
                                                             (float *)workspace, plan, batch, T, d_inner));
    }
    MRS_DISPATCH_DTYPE(dtype, T_, return launch_seq<T_>(st, s4d, gate_mode, h, y, delta, u, B, C, bc_stride, a_neg, D, gate, batch, T, d_inner, d_state));
    return MRS_OK;
}

extern "C" int mrs_ssm_scan_fwd(void *stream, int dtype, float *h, void *y, const void *delta,
                                const void *u, const void *B, const void *C, const float *a_neg,
                                const float *D, int batch, int T, int d_inner, int d_state) {
    return mrs_ssm_scan_fwd_ex(stream, dtype, h, y, delta, u, B, C, d_state, a_neg, D, nullptr,
                               MRS_GATE_NONE, nullptr, 0, batch, T, d_inner, d_state);
}
