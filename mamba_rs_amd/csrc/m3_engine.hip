// Mamba-3 SISO backbone, decode step (GpuMamba3Backbone::step, src/mamba3_siso/gpu/inference.rs:1487-1671).
//
// The reference's T = 1 layer is ten phases / fourteen launches (step_layer_kernels, inference.rs:506-1000:
// residual copy, RMSNorm, in_proj SGEMM, m3_split, bcnorm x2, bc_bias_add x2, angle_dt, rope, compute_abg,
// m3_step, gate, out_proj SGEMM, residual add).  Every one of them is launch-bound at decode batch sizes, so
// here a layer is THREE kernels:
//   1. in_proj on round(residual * norm_w) with the 1/rms row scale in the epilogue (skinny GEMM, f32 output:
//      dt, A, trap and the angles stay in f32 whatever the storage type);
//   2. m3_layer_step_kernel, one workgroup per (batch row, head): the 8-way split is just offsets into the
//      projection row; B/C RMSNorm + bias, softplus / heavy-tail / sigmoid, the angle accumulation (f64, wrapped
//      to [0, 2 pi)) and rotation, alpha/beta/gamma, the trapezoidal state update with the state row in
//      registers, y = H q + D x, and the SiLU gate (optionally RMSNormGated over the head) -- the formulas of
//      mamba3_layer_step (src/mamba3_siso/cpu/inference.rs:68-258) and kernels/mamba3_ops.cu;
//   3. out_proj with the residual add, the next layer's pre-scaled operand and row sums of squares as epilogue.
// Shapes the skinny GEMM does not take (f32 storage above four rows among them) run RMSNorm + rocBLAS GEMMs around the same step kernel.
#include "common.hpp"
#include "gemm_tune.hpp"
#include <stdlib.h>
#include "glue.hpp"
#include "m3_math.hpp"
#include <rocblas/rocblas.h>
#include <new>
#include <vector>

namespace mrs {

// One workgroup per (batch row, head); blockDim.x = hd * LG, LG = ds / 4 lanes per state row.
// proj: [batch, ip] f32 = [z:di | x:di | B:ng*ds | C:ng*ds | dd_dt:nh | dd_A:nh | trap:nh | angles:nr]
// gated: [batch, di] activation type (out_proj's operand).
template <typename T, int LG>
__global__ __launch_bounds__(1024) void m3_layer_step_kernel(
    float *__restrict__ ssm, float *__restrict__ kst, float *__restrict__ vst, float *__restrict__ angle,
    T *__restrict__ gated, const float *__restrict__ proj, int64_t ip, const float *__restrict__ dt_bias,
    const float *__restrict__ bnw, const float *__restrict__ cnw, const float *__restrict__ b_bias,
    const float *__restrict__ c_bias, const float *__restrict__ Dp, const float *__restrict__ ngw, int nh, int hd, int ng,
    int nr, float a_floor, float eps, int outproj_norm, int gated_mt) {
    constexpr int ds = 4 * LG;
    __shared__ float kl[ds], ql[ds], red[16];
    const int b = blockIdx.x / nh, h = blockIdx.x - b * nh;
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int p = tid / LG, g = tid % LG;
    const int di = nh * hd;
    const int grp = h / (nh / ng);
    const int64_t bh = (int64_t)b * nh + h;
    const float *row = proj + (int64_t)b * ip;
    const float *zr = row, *xr = row + di, *braw = row + 2 * di + (int64_t)grp * ds, *craw = row + 2 * di + (int64_t)(ng + grp) * ds;
    const float *sc = row + 2 * di + 2 * (int64_t)ng * ds;   // dd_dt | dd_A | trap | angles
    // Every global load of the kernel up front -- none depends on another -- so that the body below costs one memory
    // round trip, not one per phase; the barriers between the phases publish LDS only (lds_barrier) and leave loads in flight.
    float *Hrow = ssm + (bh * hd + p) * ds + 4 * g;
    float4 H = *reinterpret_cast<const float4 *>(Hrow);
    const float4 kp = *reinterpret_cast<const float4 *>(kst + bh * ds + 4 * g);
    const float vp = vst[bh * hd + p];
    const float xv = xr[h * hd + p];
    const float zi = zr[h * hd + p];
    const float ngv = outproj_norm ? ngw[h * hd + p] : 1.0f;
    const float Dh = Dp[h];
    const float s_dt = sc[h], s_dtb = dt_bias[h], s_A = sc[nh + h], s_tr = sc[2 * nh + h];
    const bool own_n = tid < ds, own_a = tid < nr;   // blockDim.x >= d_state (headdim >= 4)
    float bv_raw = 0.0f, cv_raw = 0.0f, bn = 0.0f, cn = 0.0f, bb_ = 0.0f, cb_ = 0.0f, ang_old = 0.0f, ang_in = 0.0f;
    if (own_n) {
        bv_raw = braw[tid]; cv_raw = craw[tid]; bn = bnw[tid]; cn = cnw[tid];
        bb_ = b_bias[(int64_t)h * ds + tid]; cb_ = c_bias[(int64_t)h * ds + tid];
    }
    if (own_a) { ang_old = angle[bh * nr + tid]; ang_in = sc[3 * nh + tid]; }

    // ---- B/C RMSNorm over d_state (bcnorm_fwd, ops/norms.rs:50-80) + per-head bias ----
    float ssb = bv_raw * bv_raw, ssc = cv_raw * cv_raw;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) { ssb += __shfl_xor(ssb, m, kWave); ssc += __shfl_xor(ssc, m, kWave); }
    // only the first ceil(ds / 64) waves hold non-zero partial sums; every wave writes its own (zero) slot
    const int wv = tid >> 6, nw = (nthr + 63) >> 6;
    if ((tid & 63) == 0 && wv < 8) { red[wv] = ssb; red[8 + wv] = ssc; }
    lds_barrier();
    float sb = 0.0f, scc = 0.0f;
    for (int i = 0; i < min(nw, 8); i++) { sb += red[i]; scc += red[8 + i]; }
    const float invb = 1.0f / sqrtf(sb / (float)ds + eps), invc = 1.0f / sqrtf(scc / (float)ds + eps);
    // per-head scalars (m3_split + compute_abg, kernels/mamba3_ops.cu:72-160, 735-753)
    const float dtv = softplus20(s_dt + s_dtb);
    if (own_n) {
        kl[tid] = bv_raw * invb * bn + bb_;
        ql[tid] = cv_raw * invc * cn + cb_;
    }
    lds_barrier();
    // ---- angle accumulation + rotation of the first 2*nr coordinates (angle_dt_fwd_batch + rope_fwd) ----
    if (own_a) {
        const int a = tid;
        const float delta = tanhf(ang_in) * kPi * dtv;
        const float an = (float)wrap_2pi((double)ang_old + (double)delta);
        angle[bh * nr + a] = an;
        float sn, cs;
        sincosf(an, &sn, &cs);
        const float b0 = kl[2 * a], b1 = kl[2 * a + 1], c0 = ql[2 * a], c1 = ql[2 * a + 1];
        kl[2 * a] = cs * b0 - sn * b1; kl[2 * a + 1] = sn * b0 + cs * b1;
        ql[2 * a] = cs * c0 - sn * c1; ql[2 * a + 1] = sn * c0 + cs * c1;
    }
    __syncthreads();   // a full barrier: every lane's read of the previous k_state has returned before the write at the end
    // ---- alpha / beta / gamma ----
    const float a_val = fminf(-heavy_tail(s_A), -a_floor);
    const float trap = sigmoidf_fast(s_tr);
    const float al = fast_exp2(a_val * dtv * kLog2e);
    const float be = al * dtv * (1.0f - trap), ga = trap * dtv;
    // ---- trapezoidal update of this lane's four states, y = H q + D x ----
    const float4 kc = *reinterpret_cast<const float4 *>(&kl[4 * g]);
    const float4 qc = *reinterpret_cast<const float4 *>(&ql[4 * g]);
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
    const float yv = fmaf(Dh, xv, acc);
    *reinterpret_cast<float4 *>(Hrow) = H;
    // ---- gate: y * silu(z), or RMSNormGated over the head first (rmsnorm_gated_forward, ops/norms.rs:84-114) ----
    float inv_y = 1.0f;
    if (outproj_norm) {
        float sq = (g == 0) ? yv * yv : 0.0f;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) sq += __shfl_xor(sq, m, kWave);
        if ((tid & 63) == 0) red[wv & 15] = sq;   // (every lane read red before the full barrier above)
        lds_barrier();
        float tot = 0.0f;
        for (int i = 0; i < min(nw, 16); i++) tot += red[i];
        inv_y = 1.0f / sqrtf(tot / (float)hd + eps);
    }
    if (g == 0) {
        const float o = outproj_norm ? yv * inv_y * ngv * silu(zi) : yv * silu(zi);
        // gated_mt != 0: out_proj reads its operand in tile order (tiled_a_index, gated_mt row tiles)
        Store<T>::st(gated + (gated_mt ? tiled_a_index(b, h * hd + p, gated_mt) : (int64_t)b * di + h * hd + p), o);
        vst[bh * hd + p] = xv;
    }
    // every lane has read the previous k_state (kp) at the top; the full barrier after the rotation orders those reads before this write
    if (p == 0) *reinterpret_cast<float4 *>(kst + bh * ds + 4 * g) = kc;
}

// ---- prefill glue ---------------------------------------------------------------------------------
// Four kernels in front of the chunked scan (the reference's m3_split, bcnorm_fwd x2, bc_bias_add x2, angle_dt_fwd,
// rope_fwd, kernels/mamba3_ops.cu:72-650):
//   m3_scalars_kernel     row-parallel: dt = softplus(dd_dt + bias), a = min(-heavy_tail(dd_A), -a_floor),
//                         trap = sigmoid(raw), and tanh(angle_raw) * pi per rope pair;
//   m3_angle_sums/apply   the rotation angle of (head, pair) at step t is the initial angle plus the running sum over
//                         time of (tanh * pi) * dt_h (angle_dt_fwd is sequential over T per thread): here T is cut into
//                         segments -- per-segment sums, the segments before folded in, then the running sums inside
//                         each segment -- in f64, wrapped to [0, 2 pi);
//   m3_kq_kernel          row-parallel: B/C RMSNorm + per-head bias + rotation -> K, Q; x -> activation type.
// Time segments of the prefill's angle scan (workgroups per batch row).  Every workgroup reads the sums of the segments
// before its own, so more segments mean more reads: at batch 4 x 4096 the two launches took 35 us with 32 segments,
// 25 us with 64, 30 us with 128.
constexpr int kAngleSegs = 64;
// One workgroup per kScalarRows consecutive rows, a thread per (row, j) with j fastest: j < nh -> the head scalars, j >= nh -> rope
// pair j - nh.  When the scan wants its per-head inputs with the steps of a head next to each other (dtT, aT, trapT:
// [batch, nh, T]) the tile is turned in LDS, so those stores are runs of kScalarRows floats.  Few rows per workgroup: every
// phase is then a single trip with all of its loads in flight at once (64 rows per workgroup, two to five dependent trips
// per phase: 13.9 us; the work itself is a few microseconds).
// bcn_out (optional, one group at d_state 64): the normalised and weighted B | C rows for the scan that forms K and Q
// itself -- out[row] = [B * rsqrt(mean(B^2) + eps) * bnw | C * rsqrt(mean(C^2) + eps) * cnw] (bcnorm_fwd, ops/norms.rs:50-80),
// formed in f32 from the f32 projection and stored in the activation type, as the reference's bcnorm_fwd_{bf16,f16} stores
// them (kernels/mamba3_ops.cu:1193-1230): every head's workgroup reads these rows for every chunk, and at 16 bits they are
// half the cache lines.  A wave per row, a lane per coordinate; the per-head bias and the rotation happen where the tiles
// are built.  (As a launch of its own this took 5.4 us, nearly all of it the fixed cost of a launch.)
constexpr int kScalarRows = 16;
template <typename T>
__global__ __launch_bounds__(1024) void m3_scalars_kernel(float *__restrict__ dt_out, float *__restrict__ a_out, float *__restrict__ trap_out,
                                                         float *__restrict__ tanhpi_out, float *__restrict__ dtT, float *__restrict__ aT,
                                                         float *__restrict__ trapT, const float *__restrict__ proj, int64_t ip,
                                                         const float *__restrict__ dt_bias, int64_t rows, int Tlen, int nh, int nr, int sc_off,
                                                         float a_floor, T *__restrict__ bcn_out, const float *__restrict__ bc, int64_t ldbc,
                                                         const float *__restrict__ bnw, const float *__restrict__ cnw, float eps) {
    extern __shared__ float turned[];   // [3][nh][kScalarRows + 1]
    constexpr int R = kScalarRows;
    const int64_t r0 = (int64_t)blockIdx.x * R;
    const int per = nh + nr;
    for (int i = threadIdx.x; i < R * per; i += (int)blockDim.x) {
        const int rl = i / per, j = i - rl * per;
        const int64_t r = r0 + rl;
        if (r >= rows) continue;
        const float *sc = proj + r * ip + sc_off;
        if (j < nh) {
            const float d = softplus20(sc[j] + dt_bias[j]);
            const float a = fminf(-heavy_tail(sc[nh + j]), -a_floor);
            const float tr = sigmoidf_fast(sc[2 * nh + j]);
            dt_out[r * nh + j] = d;
            a_out[r * nh + j] = a;
            trap_out[r * nh + j] = tr;
            if (dtT) {
                turned[(0 * nh + j) * (R + 1) + rl] = d;
                turned[(1 * nh + j) * (R + 1) + rl] = a;
                turned[(2 * nh + j) * (R + 1) + rl] = tr;
            }
        } else {
            tanhpi_out[r * nr + (j - nh)] = tanhf(sc[3 * nh + (j - nh)]) * kPi;
        }
    }
    if (bcn_out) {
        constexpr int ds = 64;
        const int w = threadIdx.x >> 6, l = threadIdx.x & 63, nw = (int)blockDim.x >> 6;
        for (int rl = w; rl < R; rl += nw) {
            const int64_t r = r0 + rl;
            if (r >= rows) break;   // whole waves
            const float b = bc[r * ldbc + l], c = bc[r * ldbc + ds + l];
            float ssb = b * b, ssc = c * c;
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) { ssb += __shfl_xor(ssb, m, kWave); ssc += __shfl_xor(ssc, m, kWave); }
            const float ib = 1.0f / sqrtf(ssb / (float)ds + eps), ic = 1.0f / sqrtf(ssc / (float)ds + eps);
            Store<T>::st(bcn_out + r * (2 * ds) + l, b * ib * bnw[l]);
            Store<T>::st(bcn_out + r * (2 * ds) + ds + l, c * ic * cnw[l]);
        }
    }
    if (!dtT) return;
    __syncthreads();
    for (int i = threadIdx.x; i < 3 * nh * R; i += (int)blockDim.x) {
        const int rl = i % R, hj = i / R, arr = hj / nh, h = hj - arr * nh;
        const int64_t r = r0 + rl;
        if (r >= rows) continue;
        const int64_t b = r / Tlen, t = r - b * Tlen;
        float *dst = arr == 0 ? dtT : (arr == 1 ? aT : trapT);
        dst[(b * nh + h) * Tlen + t] = turned[hj * (R + 1) + rl];
    }
}

// Two launches over a grid of (batch row, time segment) workgroups; thread j of a workgroup owns entry j = h * nr + a of
// the [nh][nr] angle row, so every load and store of a wave is one contiguous piece of a row (a thread per (pair,
// segment) with the pairs of one head per workgroup read and wrote 64-byte pieces a row apart: 33 us for 25 MB).
//   sums:  seg_sum[b][seg][j] = sum over the segment of (tanh * pi)[t][a] * dt[t][h] (f64); segment 0 also snapshots
//          the entering angles, which the last segment of the second launch overwrites;
//   apply: start = entering angle advanced over the segments before (wrapped after every segment), then the running
//          sums inside the segment, wrapped after every step; angle_out [rows][nh][nr] f32 (or head-major, see below).
__global__ __launch_bounds__(1024) void m3_angle_sums_kernel(double *__restrict__ seg_sum, float *__restrict__ snap,
                                                             const float *__restrict__ angle_state, const float *__restrict__ dt,
                                                             const float *__restrict__ tanhpi, int Tlen, int nh, int nr, int nsegs) {
    const int b = blockIdx.x / nsegs, seg = blockIdx.x - b * nsegs, per = nh * nr;
    const int seglen = (Tlen + nsegs - 1) / nsegs;
    const int t0 = min(Tlen, seg * seglen), t1 = min(Tlen, t0 + seglen);
    for (int j = threadIdx.x; j < per; j += blockDim.x) {
        const int h = j / nr, a = j - h * nr;
        const float *dp = dt + (int64_t)b * Tlen * nh + h;
        const float *tp = tanhpi + (int64_t)b * Tlen * nr + a;
        double sum = 0.0;
        // the operands of the next group of 8 steps are requested before the current group is added up
        float xa[8], xb[8], na[8], nb[8];
        auto request = [&](float (&a8)[8], float (&b8)[8], int tg) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int t = max(t0, min(tg + i, t1 - 1));
                a8[i] = tp[(int64_t)t * nr];
                b8[i] = dp[(int64_t)t * nh];
            }
        };
        if (t0 < t1) request(xa, xb, t0);
        for (int tg = t0; tg < t1; tg += 8) {
            request(na, nb, tg + 8);
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (tg + i < t1) sum += (double)(xa[i] * xb[i]);
#pragma unroll
            for (int i = 0; i < 8; i++) { xa[i] = na[i]; xb[i] = nb[i]; }
        }
        seg_sum[((int64_t)b * nsegs + seg) * per + j] = sum;
        if (seg == 0) snap[(int64_t)b * per + j] = angle_state[(int64_t)b * per + j];
    }
}

__global__ __launch_bounds__(1024) void m3_angle_apply_kernel(float *__restrict__ angle_out, float *__restrict__ angle_state,
                                                              const double *__restrict__ seg_sum, const float *__restrict__ snap,
                                                              const float *__restrict__ dt, const float *__restrict__ tanhpi, int Tlen,
                                                              int nh, int nr, int nsegs, int head_major) {
    const int b = blockIdx.x / nsegs, seg = blockIdx.x - b * nsegs, per = nh * nr;
    const int seglen = (Tlen + nsegs - 1) / nsegs;
    const int t0 = min(Tlen, seg * seglen), t1 = min(Tlen, t0 + seglen);
    for (int j = threadIdx.x; j < per; j += blockDim.x) {
        const int h = j / nr, a = j - h * nr;
        const float *dp = dt + (int64_t)b * Tlen * nh + h;
        const float *tp = tanhpi + (int64_t)b * Tlen * nr + a;
        // A dependent f64 operation costs tens of cycles and a wrap is half a dozen of them, so wraps stay out of the
        // serial chains: the segments before this one are summed unwrapped on four independent accumulators and wrapped
        // once, and inside the segment the chain is the running sum alone, every output wrapped on its own (equal to
        // wrapping after every step up to f64 rounding: the angles are only defined modulo 2 pi).
        double p4[4] = {0.0, 0.0, 0.0, 0.0};
        for (int s0 = 0; s0 < seg; s0 += 32) {
            double v[32];
#pragma unroll
            for (int i = 0; i < 32; i++) v[i] = s0 + i < seg ? seg_sum[((int64_t)b * nsegs + s0 + i) * per + j] : 0.0;
#pragma unroll
            for (int i = 0; i < 32; i++) p4[i & 3] += v[i];
        }
        double acc = wrap_2pi((double)snap[(int64_t)b * per + j] + ((p4[0] + p4[1]) + (p4[2] + p4[3])));
        // angle_out [rows][nh][nr], or with the steps of a head next to each other: [batch][nh][T][nr]
        float *out = angle_out + (head_major ? ((int64_t)b * nh + h) * Tlen * nr + a : (int64_t)b * Tlen * per + j);
        const int out_step = head_major ? nr : per;
        float xa[8], xb[8], na[8], nb[8];
        auto request = [&](float (&a8)[8], float (&b8)[8], int tg) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int t = max(t0, min(tg + i, t1 - 1));
                a8[i] = tp[(int64_t)t * nr];
                b8[i] = dp[(int64_t)t * nh];
            }
        };
        if (t0 < t1) request(xa, xb, t0);
        for (int tg = t0; tg < t1; tg += 8) {
            request(na, nb, tg + 8);   // the next group's operands, before this group's chain
            double run[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                acc += tg + i < t1 ? (double)(xa[i] * xb[i]) : 0.0;
                run[i] = acc;
            }
#pragma unroll
            for (int i = 0; i < 8; i++) { xa[i] = na[i]; xb[i] = nb[i]; }
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (tg + i < t1) out[(int64_t)(tg + i) * out_step] = (float)wrap_2pi(run[i]);
            acc = wrap_2pi(acc);   // once per group: keeps the running sum small
        }
        if (seg == nsegs - 1) angle_state[(int64_t)b * per + j] = (float)acc;
    }
}

// one workgroup (256 threads) per row.  bulk: rows of ldb elements [z:di | x:di | ...] in the activation type; bc: rows
// of ldbc f32 [B:ng*ds | C:ng*ds | ...] (the projection keeps them in f32, as the decode step sees them); xout may be
// null (x is then read in place by the scan).
template <typename T>
__global__ __launch_bounds__(256) void m3_kq_kernel(
    T *__restrict__ Kout, T *__restrict__ Qout, T *__restrict__ xout, const T *__restrict__ bulk, int64_t ldb,
    const float *__restrict__ bc, int64_t ldbc, const float *__restrict__ angle, const float *__restrict__ bnw, const float *__restrict__ cnw,
    const float *__restrict__ b_bias, const float *__restrict__ c_bias, int nh, int hd, int ng, int ds, int nr, float eps) {
    extern __shared__ float smem[];
    const int di = nh * hd, ngds = ng * ds;
    float *bn = smem, *cn = bn + ngds, *inv = cn + ngds;
    const int64_t r = blockIdx.x;
    const T *row = bulk + r * ldb;
    const float *bcr = bc + r * ldbc;
    const int tid = threadIdx.x;
    for (int i = tid; i < ngds; i += 256) { bn[i] = bcr[i]; cn[i] = bcr[ngds + i]; }
    __syncthreads();
    // one wave-sized slice per (B or C, group): 2*ng reductions of ds values
    {
        const int w = tid >> 6, l = tid & 63;
        for (int q = w; q < 2 * ng; q += 4) {
            const float *v = (q < ng ? bn : cn) + (q % ng) * ds;
            float ss = 0.0f;
            for (int n = l; n < ds; n += 64) ss = fmaf(v[n], v[n], ss);
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
            if (l == 0) inv[q] = 1.0f / sqrtf(ss / (float)ds + eps);
        }
    }
    __syncthreads();
    // four consecutive state coordinates (two rotation pairs) per thread and trip: 16-byte reads, 8-byte stores
    const int hpg = nh / ng, quarter = ds / 4;
    struct alignas(4 * sizeof(T)) V4 { T v[4]; };
    for (int i = tid; i < nh * quarter; i += 256) {
        const int h = i / quarter, j4 = i - h * quarter, g = h / hpg, n = 4 * j4;
        const float4 bw = *reinterpret_cast<const float4 *>(bnw + n), cw = *reinterpret_cast<const float4 *>(cnw + n);
        const float4 bb4 = *reinterpret_cast<const float4 *>(b_bias + h * ds + n), cb4 = *reinterpret_cast<const float4 *>(c_bias + h * ds + n);
        const float ib = inv[g], ic = inv[ng + g];
        float k[4] = {bn[g * ds + n] * ib * bw.x + bb4.x, bn[g * ds + n + 1] * ib * bw.y + bb4.y, bn[g * ds + n + 2] * ib * bw.z + bb4.z,
                      bn[g * ds + n + 3] * ib * bw.w + bb4.w};
        float q[4] = {cn[g * ds + n] * ic * cw.x + cb4.x, cn[g * ds + n + 1] * ic * cw.y + cb4.y, cn[g * ds + n + 2] * ic * cw.z + cb4.z,
                      cn[g * ds + n + 3] * ic * cw.w + cb4.w};
#pragma unroll
        for (int pr = 0; pr < 2; pr++) {
            const int j = 2 * j4 + pr;
            if (j < nr) {
                float s_, c_;
                sincosf(angle[(r * nh + h) * nr + j], &s_, &c_);
                const float k0 = k[2 * pr], k1 = k[2 * pr + 1], q0 = q[2 * pr], q1 = q[2 * pr + 1];
                k[2 * pr] = c_ * k0 - s_ * k1; k[2 * pr + 1] = s_ * k0 + c_ * k1;
                q[2 * pr] = c_ * q0 - s_ * q1; q[2 * pr + 1] = s_ * q0 + c_ * q1;
            }
        }
        V4 kv, qv;
#pragma unroll
        for (int e = 0; e < 4; e++) { Store<T>::st(&kv.v[e], k[e]); Store<T>::st(&qv.v[e], q[e]); }
        *reinterpret_cast<V4 *>(Kout + (r * nh + h) * ds + n) = kv;
        *reinterpret_cast<V4 *>(Qout + (r * nh + h) * ds + n) = qv;
    }
    if (xout)   // a dense copy of x for scan routes that cannot read it in place
        for (int i = tid; i < di; i += 256) xout[r * di + i] = row[di + i];
}

// The same for one group (ngroups == 1), a wave per row and no LDS: every lane forms the row's two RMS values itself
// (strided sums + a butterfly, the same order of additions as above), so nothing waits at a barrier and the operands
// of several items are in flight together.  Four rows per workgroup.
template <typename T>
__global__ __launch_bounds__(256) void m3_kq_rows_kernel(
    T *__restrict__ Kout, T *__restrict__ Qout, T *__restrict__ xout, const T *__restrict__ bulk, int64_t ldb,
    const float *__restrict__ bc, int64_t ldbc, const float *__restrict__ angle, const float *__restrict__ bnw, const float *__restrict__ cnw,
    const float *__restrict__ b_bias, const float *__restrict__ c_bias, int64_t rows, int nh, int hd, int ds, int nr, float eps) {
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + w;
    if (r >= rows) return;   // whole waves leave; the kernel has no barrier
    const int di = nh * hd;
    const T *row = bulk + r * ldb;
    const float *Bp = bc + r * ldbc, *Cp = Bp + ds;
    float ssb = 0.0f, ssc = 0.0f;
    for (int n = l; n < ds; n += 64) {
        const float b = Bp[n], c = Cp[n];
        ssb = fmaf(b, b, ssb); ssc = fmaf(c, c, ssc);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) { ssb += __shfl_xor(ssb, m, kWave); ssc += __shfl_xor(ssc, m, kWave); }
    const float ib = 1.0f / sqrtf(ssb / (float)ds + eps), ic = 1.0f / sqrtf(ssc / (float)ds + eps);
    const int quarter = ds / 4, items = nh * quarter;
    struct alignas(4 * sizeof(T)) V4 { T v[4]; };
    constexpr int kTrips = 3;   // items of a lane whose operands are requested together
    for (int i0 = l; i0 < items; i0 += 64 * kTrips) {
        float4 bv[kTrips], cv[kTrips];
        float4 bw[kTrips], cw[kTrips], bb4[kTrips], cb4[kTrips];
        float ang[kTrips][2];
#pragma unroll
        for (int t = 0; t < kTrips; t++) {
            const int i = min(i0 + 64 * t, items - 1);   // past the end: an in-range item, computed and dropped
            const int h = i / quarter, j4 = i - h * quarter, n = 4 * j4;
            bv[t] = *reinterpret_cast<const float4 *>(Bp + n); cv[t] = *reinterpret_cast<const float4 *>(Cp + n);
            bw[t] = *reinterpret_cast<const float4 *>(bnw + n); cw[t] = *reinterpret_cast<const float4 *>(cnw + n);
            bb4[t] = *reinterpret_cast<const float4 *>(b_bias + h * ds + n); cb4[t] = *reinterpret_cast<const float4 *>(c_bias + h * ds + n);
#pragma unroll
            for (int pr = 0; pr < 2; pr++) ang[t][pr] = 2 * j4 + pr < nr ? angle[(r * nh + h) * nr + 2 * j4 + pr] : 0.0f;
        }
#pragma unroll
        for (int t = 0; t < kTrips; t++) {
            const int i = i0 + 64 * t;
            if (i < items) {
                const int h = i / quarter, j4 = i - h * quarter, n = 4 * j4;
                float k[4] = {bv[t].x * ib * bw[t].x + bb4[t].x, bv[t].y * ib * bw[t].y + bb4[t].y,
                              bv[t].z * ib * bw[t].z + bb4[t].z, bv[t].w * ib * bw[t].w + bb4[t].w};
                float q[4] = {cv[t].x * ic * cw[t].x + cb4[t].x, cv[t].y * ic * cw[t].y + cb4[t].y,
                              cv[t].z * ic * cw[t].z + cb4[t].z, cv[t].w * ic * cw[t].w + cb4[t].w};
#pragma unroll
                for (int pr = 0; pr < 2; pr++) {
                    if (2 * j4 + pr < nr) {
                        float s_, c_;
                        if constexpr (sizeof(T) == 2) {
                            // angles lie in [0, 2 pi): the hardware sine / cosine (absolute error of the order of 1e-6) is
                            // far inside what a 16-bit K or Q can hold
                            s_ = __sinf(ang[t][pr]); c_ = __cosf(ang[t][pr]);
                        } else {
                            sincosf(ang[t][pr], &s_, &c_);
                        }
                        const float k0 = k[2 * pr], k1 = k[2 * pr + 1], q0 = q[2 * pr], q1 = q[2 * pr + 1];
                        k[2 * pr] = c_ * k0 - s_ * k1; k[2 * pr + 1] = s_ * k0 + c_ * k1;
                        q[2 * pr] = c_ * q0 - s_ * q1; q[2 * pr + 1] = s_ * q0 + c_ * q1;
                    }
                }
                V4 kv, qv;
#pragma unroll
                for (int e = 0; e < 4; e++) { Store<T>::st(&kv.v[e], k[e]); Store<T>::st(&qv.v[e], q[e]); }
                *reinterpret_cast<V4 *>(Kout + (r * nh + h) * ds + n) = kv;
                *reinterpret_cast<V4 *>(Qout + (r * nh + h) * ds + n) = qv;
            }
        }
    }
    if (xout)
        for (int i = l; i < di; i += 64) xout[r * di + i] = row[di + i];
}

// gated = y * silu(z) as a plain stream: a thread owns 16 bytes (8 values of 16-bit storage) of four consecutive rows and
// requests all eight vectors before it computes -- enough bytes in flight per wave that the launch is a round or two of
// waves rather than six, each of which lasts a memory round trip (one vector per thread: 24.5 us for the 75 MB of
// batch 4 x 4096 x 1536, as slow as the loop over a row it replaced).
constexpr int kGateRows = 4;
template <typename T>
__global__ __launch_bounds__(256) void m3_gate_silu_kernel(T *__restrict__ gated, const T *__restrict__ y, const T *__restrict__ bulk,
                                                           int64_t ldb, int64_t rows, int di) {
    constexpr int V = 16 / (int)sizeof(T);
    const int per_row = di / V;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t rg = i / per_row;                       // group of kGateRows rows
    const int c = (int)(i - rg * per_row) * V;
    const int64_t r0 = rg * kGateRows;
    if (r0 >= rows) return;
    struct alignas(16) V16 { T v[V]; };
    V16 zv[kGateRows], yv[kGateRows];
#pragma unroll
    for (int k = 0; k < kGateRows; k++) {
        const int64_t r = min(r0 + k, rows - 1);
        zv[k] = *reinterpret_cast<const V16 *>(bulk + r * ldb + c);
        yv[k] = *reinterpret_cast<const V16 *>(y + r * di + c);
    }
#pragma unroll
    for (int k = 0; k < kGateRows; k++) {
        if (r0 + k >= rows) break;
#pragma unroll
        for (int e = 0; e < V; e++) Store<T>::st(&yv[k].v[e], Store<T>::ld(&yv[k].v[e]) * silu(Store<T>::ld(&zv[k].v[e])));
        *reinterpret_cast<V16 *>(gated + (r0 + k) * di + c) = yv[k];
    }
}

// gated[row, i] = y * silu(z), or RMSNormGated over each head first; z = the first d_inner elements of the bulk row.
// One workgroup (256 threads) per row, a wave per head at a time for the normalised form.
template <typename T>
__global__ __launch_bounds__(256) void m3_gate_kernel(T *__restrict__ gated, const T *__restrict__ y, const T *__restrict__ bulk,
                                                      int64_t ldb, const float *__restrict__ ngw, int nh, int hd, float eps, int outproj_norm) {
    const int64_t r = blockIdx.x;
    const int di = nh * hd;
    const T *z = bulk + r * ldb;
    if (!outproj_norm) {
        if ((di & 3) == 0 && (ldb & 3) == 0) {   // four elements per thread and trip
            struct alignas(4 * sizeof(T)) V4 { T v[4]; };
            for (int i = threadIdx.x; i < di / 4; i += 256) {
                const V4 zv = *reinterpret_cast<const V4 *>(z + 4 * i);
                V4 yv = *reinterpret_cast<const V4 *>(y + r * di + 4 * i);
#pragma unroll
                for (int e = 0; e < 4; e++) Store<T>::st(&yv.v[e], Store<T>::ld(&yv.v[e]) * silu(Store<T>::ld(&zv.v[e])));
                *reinterpret_cast<V4 *>(gated + r * di + 4 * i) = yv;
            }
        } else {
            for (int i = threadIdx.x; i < di; i += 256) Store<T>::st(gated + r * di + i, Store<T>::ld(y + r * di + i) * silu(Store<T>::ld(z + i)));
        }
        return;
    }
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    for (int h = w; h < nh; h += 4) {
        float ss = 0.0f;
        for (int p = l; p < hd; p += 64) { const float v = Store<T>::ld(y + r * di + h * hd + p); ss = fmaf(v, v, ss); }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
        const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
        for (int p = l; p < hd; p += 64) {
            const int i = h * hd + p;
            Store<T>::st(gated + r * di + i, Store<T>::ld(y + r * di + i) * inv * ngw[i] * silu(Store<T>::ld(z + i)));
        }
    }
}

}  // namespace mrs

using namespace mrs;

#define MRS_HIP(expr)                                                                        \
    do { hipError_t e_ = (expr); if (e_ != hipSuccess) return fail(MRS_E_HIP, "%s: %s", #expr, hipGetErrorString(e_)); } while (0)
#define MRS_TRY(expr) do { int rc_ = (expr); if (rc_) return rc_; } while (0)
#define MRS_BLAS(expr)                                                                        \
    do { rocblas_status s_ = (expr); if (s_ != rocblas_status_success) return fail(MRS_E_HIP, "%s: rocblas status %d", #expr, (int)s_); } while (0)

namespace {

inline size_t esize3(int dtype) { return dtype == MRS_F32 ? 4 : 2; }
inline rocblas_datatype blas_type3(int dtype) {
    return dtype == MRS_F32 ? rocblas_datatype_f32_r : dtype == MRS_F16 ? rocblas_datatype_f16_r : rocblas_datatype_bf16_r;
}

struct Layer3 {
    float *norm_w, *dt_bias, *bnw, *cnw, *b_bias, *c_bias, *D, *ngw;
    void *in_proj, *out_proj;      // [K][N] storage type (library GEMM)
    void *in_proj_t, *out_proj_t;  // [N][K] copies for the skinny GEMM (null: library chain)
    void *in_proj_p, *out_proj_p;  // tiled copies (launch_tile_weight): the own chain from two rows up
};

}  // namespace

struct mrs_m3_backbone {
    mrs_m3_config cfg;
    int input_dim, batch, dtype, di, nh, ip, nr, identity_proj, device, skinny, tiled;
    hipStream_t stream;
    rocblas_handle blas;
    GemmTuner *tuner;       // vendor-kernel choice for the prefill projections (off unless asked for)
    TinyM3StepLayer *tiny_layers;   // small f32 models: the layer table of the single-launch step (null: kernel chains)
    std::vector<Layer3> layers;
    std::vector<void *> allocs;
    std::vector<void *> pf_allocs;   // the prefill scratch alone: released and re-made when the sequence length changes
    float *input_proj_w, *input_proj_b, *norm_f;
    float *ssm, *kst, *vst, *angle;          // [L][batch]...
    float *d_input, *temporal, *residual, *proj, *partials;
    void *normed, *gated, *out;
    hipGraph_t graph;
    hipGraphExec_t graph_exec;
    int graph_ready;
    // prefill scratch for sequences of pf_T steps (0: not allocated)
    int pf_T;
    float *pf_in, *pf_residual, *pf_proj, *pf_dt, *pf_a, *pf_trap, *pf_tanhpi, *pf_angle, *pf_angle_snap;
    float *pf_dtT, *pf_aT, *pf_trapT;   // [batch, nh, T] copies of dt, a, trap for the scan that forms K and Q itself
    double *pf_angle_sums;   // [batch][kAngleSegs][nh * n_rope] per-segment angle increments of the prefill
    void *pf_bcn;            // [rows][2 * d_state] normalised and weighted B | C rows (activation type) for the scan that forms K and Q itself
    void *pf_normed, *pf_bulk, *pf_x, *pf_K, *pf_Q, *pf_y, *pf_gated, *pf_out, *pf_ws;
    size_t pf_ws_bytes;
};

namespace {

int dev_alloc3(mrs_m3_backbone *bb, void **p, size_t bytes) {
    MRS_HIP(hipMalloc(p, bytes ? bytes : 16));
    bb->allocs.push_back(*p);
    return MRS_OK;
}
int upload_f32_3(mrs_m3_backbone *bb, float **dst, const float *src, size_t n) {
    MRS_TRY(dev_alloc3(bb, (void **)dst, n * sizeof(float)));
    MRS_HIP(hipMemcpyAsync(*dst, src, n * sizeof(float), hipMemcpyHostToDevice, bb->stream));
    return MRS_OK;
}
// bulk matrix: upload f32, round to the storage type on device (RNE)
int upload_bulk3(mrs_m3_backbone *bb, void **dst, const float *src, size_t n, float *stage) {
    MRS_HIP(hipMemcpyAsync(stage, src, n * sizeof(float), hipMemcpyHostToDevice, bb->stream));
    MRS_TRY(dev_alloc3(bb, dst, n * esize3(bb->dtype)));
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (bb->dtype == MRS_F32) MRS_HIP(hipMemcpyAsync(*dst, stage, n * 4, hipMemcpyDeviceToDevice, bb->stream));
    else if (bb->dtype == MRS_BF16) hipLaunchKernelGGL((cast_from_f32_kernel<bf16_t>), grid, block, 0, bb->stream, (bf16_t *)*dst, stage, (int64_t)n);
    else hipLaunchKernelGGL((cast_from_f32_kernel<f16_t>), grid, block, 0, bb->stream, (f16_t *)*dst, stage, (int64_t)n);
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return check_launch("weight cast");
}

// C[M,N] (f32 or storage type) = A[M,K] . W[K,N], row-major, f32 accumulate (library GEMM)
int gemm3(mrs_m3_backbone *bb, void *C, bool c_f32, const void *A, const void *W, int M, int N, int K) {
    const rocblas_datatype t = blas_type3(bb->dtype), ct = c_f32 ? rocblas_datatype_f32_r : t;
    return gemm_ex_tuned(bb->tuner, bb->blas, bb->stream, 0, N, M, K, W, t, N, A, t, K, C, ct, N);
}

template <typename T>
int launch_layer_step_t(mrs_m3_backbone *bb, int l) {
    const mrs_m3_config &c = bb->cfg;
    const Layer3 &lw = bb->layers[l];
    const int B = bb->batch, nh = bb->nh, hd = c.headdim, ds = c.d_state, lg = ds / 4;
    float *ssm = bb->ssm + (size_t)l * B * nh * hd * ds, *kst = bb->kst + (size_t)l * B * nh * ds;
    float *vst = bb->vst + (size_t)l * B * nh * hd, *ang = bb->angle + (size_t)l * B * nh * (bb->nr > 0 ? bb->nr : 1);
    const dim3 grid((unsigned)(B * nh)), block((unsigned)(hd * lg));
#define MRS_LG(L)                                                                                                                 \
    case L:                                                                                                                       \
        hipLaunchKernelGGL((m3_layer_step_kernel<T, L>), grid, block, 0, bb->stream, ssm, kst, vst, ang, (T *)bb->gated, bb->proj,  \
                           (int64_t)bb->ip, lw.dt_bias, lw.bnw, lw.cnw, lw.b_bias, lw.c_bias, lw.D, lw.ngw, nh, hd, c.ngroups,     \
                           bb->nr, c.a_floor, c.rms_norm_eps, c.is_outproj_norm, bb->tiled ? (B + 15) / 16 : 0);                   \
        break
    switch (lg) { MRS_LG(1); MRS_LG(2); MRS_LG(4); MRS_LG(8); MRS_LG(16); MRS_LG(32); MRS_LG(64); default: return fail(MRS_E_SHAPE, "m3 layer step: d_state %d", ds); }
#undef MRS_LG
    return check_launch("m3_layer_step_kernel");
}

int step_body3(mrs_m3_backbone *bb) {
    const mrs_m3_config &c = bb->cfg;
    if (bb->tiny_layers) {
        TinyM3StepArgs a = {};
        a.layers = bb->tiny_layers; a.input = bb->d_input;
        a.in_w = bb->identity_proj ? nullptr : bb->input_proj_w; a.in_b = bb->identity_proj ? nullptr : bb->input_proj_b;
        a.norm_f = bb->norm_f; a.ssm = bb->ssm; a.kst = bb->kst; a.vst = bb->vst; a.angle = bb->angle; a.temporal = bb->temporal;
        a.eps = c.rms_norm_eps; a.a_floor = c.a_floor; a.n_layers = c.n_layers; a.batch = bb->batch; a.input_dim = bb->input_dim;
        a.dm = c.d_model; a.di = bb->di; a.nh = bb->nh; a.hd = c.headdim; a.ds = c.d_state; a.ng = c.ngroups; a.nr = bb->nr; a.ip = bb->ip;
        a.outproj_norm = c.is_outproj_norm;
        return launch_tiny_m3_step(bb->stream, a);
    }
    const int dm = c.d_model, di = bb->di, B = bb->batch, dt = bb->dtype, L = c.n_layers, ip = bb->ip;
    const int P = (dm + 15) / 16;
    const int a_mt = bb->tiled ? (B + 15) / 16 : 0;   // the projections' operands in tile order (16-row tiles)
    // residual <- input (identity) or input . W + b
    const float *src = nullptr;
    if (bb->identity_proj) {
        if (bb->skinny) src = bb->d_input;   // the first prenorm kernel reads the input and writes the residual stream
        else MRS_HIP(hipMemcpyAsync(bb->residual, bb->d_input, (size_t)B * dm * 4, hipMemcpyDeviceToDevice, bb->stream));
    } else {
        const int64_t n = (int64_t)B * dm;
        hipLaunchKernelGGL(bias_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, bb->stream, bb->residual, bb->input_proj_b, n, dm);
        const float one = 1.0f;
        MRS_BLAS(rocblas_gemm_ex(bb->blas, rocblas_operation_none, rocblas_operation_none, dm, B, bb->input_dim, &one, bb->input_proj_w,
                                 rocblas_datatype_f32_r, dm, bb->d_input, rocblas_datatype_f32_r, bb->input_dim, &one, bb->residual,
                                 rocblas_datatype_f32_r, dm, bb->residual, rocblas_datatype_f32_r, dm, rocblas_datatype_f32_r,
                                 rocblas_gemm_algo_standard, 0, 0));
    }
    for (int l = 0; l < L; l++) {
        const Layer3 &lw = bb->layers[l];
        if (bb->skinny) {
            if (l == 0)
                MRS_TRY(launch_prenorm_rows(bb->stream, dt, bb->partials, P, bb->normed, src ? src : bb->residual, src ? bb->residual : nullptr,
                                            lw.norm_w, B, dm, a_mt));
            SkinnyEpi inp = {};
            inp.row_scale = 1; inp.partials = bb->partials; inp.n_partials = P; inp.eps = c.rms_norm_eps;
            inp.a_tiled = inp.w_tiled = a_mt ? 1 : 0;
            MRS_TRY(launch_skinny_gemm(bb->stream, dt, bb->proj, 1, ip, bb->normed, dm, a_mt ? lw.in_proj_p : lw.in_proj_t, B, ip, dm, inp));
        } else {
            MRS_TRY(launch_add_rmsnorm_any(bb->stream, dt, bb->residual, l == 0 ? nullptr : bb->out, bb->normed, false, nullptr, lw.norm_w,
                                           c.rms_norm_eps, B, dm, dm));
            MRS_TRY(gemm3(bb, bb->proj, true, bb->normed, lw.in_proj, B, ip, dm));
        }
        MRS_DISPATCH_DTYPE(dt, T_, MRS_TRY(launch_layer_step_t<T_>(bb, l)));
        if (bb->skinny) {
            SkinnyEpi outp = {};
            outp.mode = 2; outp.residual = bb->residual; outp.partials = bb->partials; outp.n_partials = P;
            outp.next_norm_w = l + 1 < L ? bb->layers[l + 1].norm_w : nullptr; outp.prenorm = bb->normed;
            outp.a_tiled = outp.w_tiled = a_mt ? 1 : 0; outp.prenorm_mt = a_mt;
            MRS_TRY(launch_skinny_gemm(bb->stream, dt, bb->out, 0, dm, bb->gated, di, a_mt ? lw.out_proj_p : lw.out_proj_t, B, dm, di, outp));
        } else {
            MRS_TRY(gemm3(bb, bb->out, false, bb->gated, lw.out_proj, B, dm, di));
        }
    }
    // final residual add (library chain) + norm_f -> temporal (f32)
    return launch_add_rmsnorm_any(bb->stream, dt, bb->residual, bb->skinny ? nullptr : bb->out, bb->temporal, true, nullptr, bb->norm_f,
                                  c.rms_norm_eps, B, dm, dm);
}

}  // namespace

extern "C" int mrs_m3_backbone_reset(mrs_m3_backbone *bb) {
    if (!bb) return fail(MRS_E_NULL, "mrs_m3_backbone_reset: null engine");
    const size_t L = bb->cfg.n_layers, B = bb->batch, nh = bb->nh, hd = bb->cfg.headdim, ds = bb->cfg.d_state, na = bb->nr > 0 ? bb->nr : 1;
    MRS_HIP(hipMemsetAsync(bb->ssm, 0, L * B * nh * hd * ds * 4, bb->stream));
    MRS_HIP(hipMemsetAsync(bb->kst, 0, L * B * nh * ds * 4, bb->stream));
    MRS_HIP(hipMemsetAsync(bb->vst, 0, L * B * nh * hd * 4, bb->stream));
    MRS_HIP(hipMemsetAsync(bb->angle, 0, L * B * nh * na * 4, bb->stream));
    return MRS_OK;
}

extern "C" void mrs_m3_backbone_destroy(mrs_m3_backbone *bb) {
    if (!bb) return;
    hipSetDevice(bb->device);
    if (bb->stream) hipStreamSynchronize(bb->stream);
    if (bb->graph_exec) hipGraphExecDestroy(bb->graph_exec);
    if (bb->graph) hipGraphDestroy(bb->graph);
    for (void *p : bb->allocs) hipFree(p);
    for (void *p : bb->pf_allocs) hipFree(p);
    gemm_tuner_destroy(bb->tuner);
    if (bb->blas) rocblas_destroy_handle(bb->blas);
    if (bb->stream) hipStreamDestroy(bb->stream);
    delete bb;
}

extern "C" int mrs_m3_backbone_create(mrs_m3_backbone **out, int gpu_ordinal, const mrs_m3_weights *w, const mrs_m3_config *cfg,
                                      int input_dim, int batch, int dtype) {
    const char *fn = "mrs_m3_backbone_create";
    if (!out || !w || !cfg || !w->layers || !w->norm_f_weight) return fail(MRS_E_NULL, "%s: null pointer", fn);
    if (dtype != MRS_F32 && dtype != MRS_F16 && dtype != MRS_BF16) return fail(MRS_E_DTYPE, "%s: dtype %d", fn, dtype);
    // Mamba3Config::validate (src/mamba3_siso/config.rs:60-131), with this library's wider headdim / d_state limits
    if (cfg->d_model < 1 || cfg->d_state < 1 || cfg->expand < 1 || cfg->headdim < 1 || cfg->ngroups < 1 || cfg->n_layers < 1)
        return fail(MRS_E_SHAPE, "%s: d_model, d_state, expand, headdim, ngroups, n_layers must be > 0", fn);
    const int64_t di64 = (int64_t)cfg->d_model * cfg->expand;
    if (di64 % cfg->headdim != 0) return fail(MRS_E_SHAPE, "%s: d_inner %lld is not a multiple of headdim %d", fn, (long long)di64, cfg->headdim);
    const int nh = (int)(di64 / cfg->headdim);
    if (nh % cfg->ngroups != 0) return fail(MRS_E_SHAPE, "%s: nheads %d is not a multiple of ngroups %d", fn, nh, cfg->ngroups);
    const int ds = cfg->d_state, lg = ds / 4;
    // one lane per four states of a row: a workgroup of headdim * d_state / 4 lanes, whole waves only
    if (ds % 4 != 0 || (lg & (lg - 1)) != 0 || lg > 64 || cfg->headdim < 4 || (int64_t)cfg->headdim * lg > 1024 || ((int64_t)cfg->headdim * lg) % 64 != 0)
        return fail(MRS_E_SHAPE, "%s: d_state must be 4 x a power of two <= 256 and headdim * d_state / 4 a multiple of 64 <= 1024 (got %d, %d)", fn, ds, cfg->headdim);
    if (cfg->n_rope_angles < 0 || 2 * cfg->n_rope_angles > ds) return fail(MRS_E_SHAPE, "%s: n_rope_angles %d outside 0..d_state/2", fn, cfg->n_rope_angles);
    if (!(cfg->a_floor > 0.0f)) return fail(MRS_E_SHAPE, "%s: a_floor must be > 0", fn);
    if (batch < 1 || input_dim < 1 || di64 > 65535 || cfg->n_layers > 4096) return fail(MRS_E_SHAPE, "%s: batch=%d input_dim=%d d_inner=%lld", fn, batch, input_dim, (long long)di64);
    const int identity = (w->input_proj_w == nullptr);
    if (identity && input_dim != cfg->d_model) return fail(MRS_E_SHAPE, "%s: identity input_proj needs input_dim == d_model", fn);
    mrs_m3_backbone *bb = new (std::nothrow) mrs_m3_backbone();
    if (!bb) return fail(MRS_E_HIP, "%s: out of host memory", fn);
    bb->cfg = *cfg; bb->input_dim = input_dim; bb->batch = batch; bb->dtype = dtype; bb->device = gpu_ordinal;
    bb->di = (int)di64; bb->nh = nh; bb->nr = cfg->n_rope_angles; bb->identity_proj = identity;
    bb->ip = 2 * bb->di + 2 * cfg->ngroups * ds + 3 * nh + bb->nr;
    bb->graph_ready = 0; bb->graph = nullptr; bb->graph_exec = nullptr; bb->input_proj_w = nullptr; bb->input_proj_b = nullptr;
    bb->pf_T = 0;
    *out = nullptr;
#define MRS_CREATE_TRY(expr) do { int rc_ = (expr); if (rc_) { mrs_m3_backbone_destroy(bb); return rc_; } } while (0)
    {
        hipError_t e = hipSetDevice(gpu_ordinal);
        if (e != hipSuccess) { delete bb; return fail(MRS_E_HIP, "hipSetDevice(%d): %s", gpu_ordinal, hipGetErrorString(e)); }
        e = hipStreamCreateWithFlags(&bb->stream, hipStreamNonBlocking);
        if (e != hipSuccess) { delete bb; return fail(MRS_E_HIP, "hipStreamCreate: %s", hipGetErrorString(e)); }
        if (rocblas_create_handle(&bb->blas) != rocblas_status_success) { hipStreamDestroy(bb->stream); delete bb; return fail(MRS_E_HIP, "rocblas_create_handle failed"); }
        rocblas_set_stream(bb->blas, bb->stream);
        bb->tuner = gemm_tuner_create();
        { const char *e = getenv("MRS_GEMM_TUNE"); gemm_tuner_enable(bb->tuner, e && atoi(e) != 0); }
        rocblas_set_pointer_mode(bb->blas, rocblas_pointer_mode_host);
    }
    const int dm = cfg->d_model, di = bb->di, ip = bb->ip, L = cfg->n_layers;
    // (above 64 rows the library chain is the faster one for this layer: 1261 vs 1318 us per step at 128 rows, 768-wide shape)
    bb->skinny = (dtype == MRS_BF16 || dtype == MRS_F16) && batch <= std::min(64, skinny_max_rows()) && dm % 32 == 0 && di % 32 == 0;
    // from two rows up the two projections run on the matrix cores and read tiled weights and tiled activation operands
    // (768-wide shape, per step, row-wise / tiled route: 282 / 302 us at 1 row, 326 / 308 at 2, 364 / 308 at 3, 368 / 314 at 4)
    { const char *e = getenv("MRS_DECODE_NO_TILED"), *m = getenv("MRS_DECODE_TILED_MIN_ROWS");
      bb->tiled = bb->skinny && (dtype == MRS_BF16 || dtype == MRS_F16) && batch >= (m ? atoi(m) : 2) && !(e && atoi(e) != 0); }
    // f32 storage: the row-wise route of the same GEMM, one to four rows
    if (dtype == MRS_F32 && batch <= 4 && dm % 128 == 0 && di % 128 == 0 && (int64_t)di * 16 <= 48 * 1024 && getenv("MRS_DECODE_NO_ROWWISE") == nullptr)
        bb->skinny = 1;
    float *stage = nullptr;
    {
        size_t big = (size_t)dm * ip;
        if ((size_t)di * dm > big) big = (size_t)di * dm;
        MRS_CREATE_TRY(dev_alloc3(bb, (void **)&stage, big * sizeof(float)));
    }
    if (!identity) {
        MRS_CREATE_TRY(upload_f32_3(bb, &bb->input_proj_w, w->input_proj_w, (size_t)input_dim * dm));
        if (w->input_proj_b) MRS_CREATE_TRY(upload_f32_3(bb, &bb->input_proj_b, w->input_proj_b, dm));
    }
    bb->layers.resize(L);
    for (int l = 0; l < L; l++) {
        const mrs_m3_layer_weights &s = w->layers[l];
        Layer3 &d = bb->layers[l];
        if (!s.norm_weight || !s.in_proj_w || !s.dt_bias || !s.b_norm_weight || !s.c_norm_weight || !s.b_bias || !s.c_bias || !s.d_param ||
            !s.norm_gate_weight || !s.out_proj_w) {
            mrs_m3_backbone_destroy(bb);
            return fail(MRS_E_NULL, "%s: layer %d has a null weight", fn, l);
        }
        MRS_CREATE_TRY(upload_f32_3(bb, &d.norm_w, s.norm_weight, dm));
        MRS_CREATE_TRY(upload_bulk3(bb, &d.in_proj, s.in_proj_w, (size_t)dm * ip, stage));
        MRS_CREATE_TRY(upload_f32_3(bb, &d.dt_bias, s.dt_bias, nh));
        MRS_CREATE_TRY(upload_f32_3(bb, &d.bnw, s.b_norm_weight, ds));
        MRS_CREATE_TRY(upload_f32_3(bb, &d.cnw, s.c_norm_weight, ds));
        MRS_CREATE_TRY(upload_f32_3(bb, &d.b_bias, s.b_bias, (size_t)nh * ds));
        MRS_CREATE_TRY(upload_f32_3(bb, &d.c_bias, s.c_bias, (size_t)nh * ds));
        MRS_CREATE_TRY(upload_f32_3(bb, &d.D, s.d_param, nh));
        MRS_CREATE_TRY(upload_f32_3(bb, &d.ngw, s.norm_gate_weight, di));
        MRS_CREATE_TRY(upload_bulk3(bb, &d.out_proj, s.out_proj_w, (size_t)di * dm, stage));
        d.in_proj_t = d.out_proj_t = nullptr;
        if (bb->skinny) {
            const size_t es = esize3(dtype);
            MRS_CREATE_TRY(dev_alloc3(bb, &d.in_proj_t, (size_t)dm * ip * es));
            MRS_CREATE_TRY(dev_alloc3(bb, &d.out_proj_t, (size_t)di * dm * es));
            MRS_CREATE_TRY(launch_transpose(bb->stream, dtype, d.in_proj_t, d.in_proj, dm, ip));
            MRS_CREATE_TRY(launch_transpose(bb->stream, dtype, d.out_proj_t, d.out_proj, di, dm));
        }
        d.in_proj_p = d.out_proj_p = nullptr;
        if (bb->tiled) {
            const size_t es = esize3(dtype);
            MRS_CREATE_TRY(dev_alloc3(bb, &d.in_proj_p, tiled_weight_elems(ip, dm) * es));
            MRS_CREATE_TRY(dev_alloc3(bb, &d.out_proj_p, tiled_weight_elems(dm, di) * es));
            MRS_CREATE_TRY(launch_tile_weight(bb->stream, dtype, d.in_proj_p, d.in_proj_t, ip, dm));
            MRS_CREATE_TRY(launch_tile_weight(bb->stream, dtype, d.out_proj_p, d.out_proj_t, dm, di));
        }
    }
    MRS_CREATE_TRY(upload_f32_3(bb, &bb->norm_f, w->norm_f_weight, dm));
    {
        // small f32 models: a step is one launch (MRS_DECODE_NO_TINY=1 keeps the kernel chains)
        const char *e = getenv("MRS_DECODE_NO_TINY");
        if (!(e && atoi(e) != 0) && tiny_m3_step_ok(dtype, input_dim, dm, di, nh, cfg->headdim, ds, cfg->ngroups, bb->nr, ip)) {
            std::vector<TinyM3StepLayer> tl((size_t)L);
            for (int l = 0; l < L; l++) {
                const Layer3 &d = bb->layers[l];
                tl[(size_t)l] = {d.norm_w, (const float *)d.in_proj, d.dt_bias, d.bnw, d.cnw, d.b_bias, d.c_bias, d.D, d.ngw, (const float *)d.out_proj};
            }
            MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->tiny_layers, (size_t)L * sizeof(TinyM3StepLayer)));
            hipError_t he = hipMemcpyAsync(bb->tiny_layers, tl.data(), (size_t)L * sizeof(TinyM3StepLayer), hipMemcpyHostToDevice, bb->stream);
            if (he == hipSuccess) he = hipStreamSynchronize(bb->stream);   // tl leaves scope below
            if (he != hipSuccess) { mrs_m3_backbone_destroy(bb); return fail(MRS_E_HIP, "%s: layer table upload: %s", fn, hipGetErrorString(he)); }
        }
    }
    const size_t B = batch, hd = cfg->headdim, na = bb->nr > 0 ? bb->nr : 1, es = esize3(dtype);
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->ssm, (size_t)L * B * nh * hd * ds * 4));
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->kst, (size_t)L * B * nh * ds * 4));
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->vst, (size_t)L * B * nh * hd * 4));
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->angle, (size_t)L * B * nh * na * 4));
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->d_input, B * input_dim * 4));
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->temporal, B * dm * 4));
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->residual, B * dm * 4));
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->proj, B * ip * 4));
    MRS_CREATE_TRY(dev_alloc3(bb, (void **)&bb->partials, B * ((dm + 15) / 16) * 4));
    const size_t B16 = bb->tiled ? (B + 15) / 16 * 16 : B;   // tiled operands come in 16-row tiles
    MRS_CREATE_TRY(dev_alloc3(bb, &bb->normed, B16 * dm * es));
    MRS_CREATE_TRY(dev_alloc3(bb, &bb->gated, B16 * di * es));
    MRS_CREATE_TRY(dev_alloc3(bb, &bb->out, B * dm * es));
    MRS_CREATE_TRY(mrs_m3_backbone_reset(bb));
    { hipError_t e = hipStreamSynchronize(bb->stream);
      if (e != hipSuccess) { mrs_m3_backbone_destroy(bb); return fail(MRS_E_HIP, "create sync: %s", hipGetErrorString(e)); } }
#undef MRS_CREATE_TRY
    *out = bb;
    return MRS_OK;
}

extern "C" int mrs_m3_backbone_step_gpu_only(mrs_m3_backbone *bb) {
    if (!bb) return fail(MRS_E_NULL, "mrs_m3_backbone_step_gpu_only: null engine");
    if (bb->graph_ready) { MRS_HIP(hipGraphLaunch(bb->graph_exec, bb->stream)); return MRS_OK; }
    return step_body3(bb);
}

extern "C" int mrs_m3_backbone_step(mrs_m3_backbone *bb, const float *input, float *output) {
    if (!bb || !input || !output) return fail(MRS_E_NULL, "mrs_m3_backbone_step: null pointer");
    MRS_HIP(hipMemcpyAsync(bb->d_input, input, (size_t)bb->batch * bb->input_dim * 4, hipMemcpyHostToDevice, bb->stream));
    MRS_TRY(mrs_m3_backbone_step_gpu_only(bb));
    MRS_HIP(hipMemcpyAsync(output, bb->temporal, (size_t)bb->batch * bb->cfg.d_model * 4, hipMemcpyDeviceToHost, bb->stream));
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}

// One eager warm step on a saved copy of the state (library handles pick their kernels), then capture the step body
// (capture_graph, src/mamba3_siso/gpu/inference.rs:1560-1600).  The capture is always ended on error.
extern "C" int mrs_m3_backbone_capture_graph(mrs_m3_backbone *bb) {
    if (!bb) return fail(MRS_E_NULL, "mrs_m3_backbone_capture_graph: null engine");
    if (bb->graph_ready) return MRS_OK;
    const size_t L = bb->cfg.n_layers, B = bb->batch, nh = bb->nh, hd = bb->cfg.headdim, ds = bb->cfg.d_state, na = bb->nr > 0 ? bb->nr : 1;
    const size_t n0 = L * B * nh * hd * ds * 4, n1 = L * B * nh * ds * 4, n2 = L * B * nh * hd * 4, n3 = L * B * nh * na * 4;
    char *save = nullptr;
    MRS_HIP(hipMalloc((void **)&save, n0 + n1 + n2 + n3));
    hipMemcpyAsync(save, bb->ssm, n0, hipMemcpyDeviceToDevice, bb->stream);
    hipMemcpyAsync(save + n0, bb->kst, n1, hipMemcpyDeviceToDevice, bb->stream);
    hipMemcpyAsync(save + n0 + n1, bb->vst, n2, hipMemcpyDeviceToDevice, bb->stream);
    hipMemcpyAsync(save + n0 + n1 + n2, bb->angle, n3, hipMemcpyDeviceToDevice, bb->stream);
    int rc = step_body3(bb);
    hipMemcpyAsync(bb->ssm, save, n0, hipMemcpyDeviceToDevice, bb->stream);
    hipMemcpyAsync(bb->kst, save + n0, n1, hipMemcpyDeviceToDevice, bb->stream);
    hipMemcpyAsync(bb->vst, save + n0 + n1, n2, hipMemcpyDeviceToDevice, bb->stream);
    hipMemcpyAsync(bb->angle, save + n0 + n1 + n2, n3, hipMemcpyDeviceToDevice, bb->stream);
    hipError_t e = hipStreamSynchronize(bb->stream);
    hipFree(save);
    if (rc) return rc;
    if (e != hipSuccess) return fail(MRS_E_HIP, "capture warm-up: %s", hipGetErrorString(e));
    MRS_HIP(hipStreamBeginCapture(bb->stream, hipStreamCaptureModeThreadLocal));
    rc = step_body3(bb);
    hipGraph_t g = nullptr;
    e = hipStreamEndCapture(bb->stream, &g);
    if (rc) { if (g) hipGraphDestroy(g); return rc; }
    if (e != hipSuccess) return fail(MRS_E_HIP, "hipStreamEndCapture: %s", hipGetErrorString(e));
    hipGraphExec_t ge = nullptr;
    e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
    if (e != hipSuccess) { hipGraphDestroy(g); return fail(MRS_E_HIP, "hipGraphInstantiate: %s", hipGetErrorString(e)); }
    bb->graph = g; bb->graph_exec = ge; bb->graph_ready = 1;
    return MRS_OK;
}

// ---- prefill -----------------------------------------------------------------------------------------
// Prefill scratch follows the sequence length of the call (the reference allocates it per call,
// src/module/gpu_lm3.rs): kept while T stays the same, released and re-made when it changes.  Not for use while a
// capture is open on the engine's stream.
static int alloc_prefill_scratch3(mrs_m3_backbone *bb, int T);
extern "C" int mrs_m3_backbone_alloc_prefill_scratch(mrs_m3_backbone *bb, int T) {
    const char *fn = "mrs_m3_backbone_alloc_prefill_scratch";
    if (!bb) return fail(MRS_E_NULL, "%s: null engine", fn);
    if (T < 1) return fail(MRS_E_SHAPE, "%s: T=%d", fn, T);
    if (bb->pf_T == T) return MRS_OK;
    auto release = [&]() {
        hipStreamSynchronize(bb->stream);   // no kernel may still be reading the old buffers
        for (void *p : bb->pf_allocs) hipFree(p);
        bb->pf_allocs.clear();
        bb->pf_T = 0; bb->pf_in = nullptr;
    };
    if (bb->pf_T) release();
    const size_t mark = bb->allocs.size();
    const int rc = alloc_prefill_scratch3(bb, T);
    bb->pf_allocs.assign(bb->allocs.begin() + mark, bb->allocs.end());
    bb->allocs.resize(mark);
    if (rc) release();
    return rc;
}

static int alloc_prefill_scratch3(mrs_m3_backbone *bb, int T) {
    const char *fn = "mrs_m3_backbone_alloc_prefill_scratch";
    const mrs_m3_config &c = bb->cfg;
    const size_t rows = (size_t)bb->batch * T, es = esize3(bb->dtype), dm = c.d_model, di = bb->di, nh = bb->nh, ds = c.d_state, ip = bb->ip;
    if ((int64_t)rows * ip > 0x7fffffffLL) return fail(MRS_E_SHAPE, "%s: batch*T*in_proj_dim exceeds i32", fn);
    if (bb->nr > 1024) return fail(MRS_E_SHAPE, "%s: more than 1024 rope pairs", fn);
    const size_t nrz = bb->nr > 0 ? bb->nr : 1;
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_in, rows * bb->input_dim * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_residual, rows * dm * 4));
    // f32 storage: the whole in_proj result; 16-bit: its f32 columns only (B, C, head scalars, angle inputs), the bulk
    // columns (z, x) live in pf_bulk
    const size_t nbulk = 2 * di;
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_proj, rows * (bb->dtype == MRS_F32 ? ip : ip - nbulk) * 4));
    MRS_TRY(dev_alloc3(bb, &bb->pf_bulk, bb->dtype == MRS_F32 ? 16 : rows * nbulk * es));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_dt, rows * nh * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_a, rows * nh * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_trap, rows * nh * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_dtT, rows * nh * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_aT, rows * nh * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_trapT, rows * nh * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_tanhpi, rows * nrz * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_angle, rows * nh * nrz * 4));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_angle_sums, (size_t)bb->batch * kAngleSegs * nh * nrz * sizeof(double)));
    MRS_TRY(dev_alloc3(bb, (void **)&bb->pf_angle_snap, (size_t)bb->batch * nh * nrz * 4));
    MRS_TRY(dev_alloc3(bb, &bb->pf_bcn, rows * 2 * ds * es));
    MRS_TRY(dev_alloc3(bb, &bb->pf_normed, rows * dm * es));
    MRS_TRY(dev_alloc3(bb, &bb->pf_x, rows * di * es));
    MRS_TRY(dev_alloc3(bb, &bb->pf_K, rows * nh * ds * es));
    MRS_TRY(dev_alloc3(bb, &bb->pf_Q, rows * nh * ds * es));
    MRS_TRY(dev_alloc3(bb, &bb->pf_y, rows * di * es));
    MRS_TRY(dev_alloc3(bb, &bb->pf_gated, rows * di * es));
    MRS_TRY(dev_alloc3(bb, &bb->pf_out, rows * dm * es));
    size_t wsb = mrs_m3_ssd_workspace_bytes(bb->batch, T, (int)nh, c.headdim, c.d_state, 64);
    const size_t abg = 3 * rows * nh * 4;   // alpha, beta, gamma for shapes the chunked kernel does not take
    if (abg > wsb) wsb = abg;
    bb->pf_ws_bytes = wsb;
    MRS_TRY(dev_alloc3(bb, &bb->pf_ws, wsb));
    bb->pf_T = T;
    return MRS_OK;
}

namespace {

template <typename T>
int launch_kq_t(mrs_m3_backbone *bb, const Layer3 &lw, int64_t rows, const void *bulk, int64_t ldb, const float *bc, int64_t ldbc, bool copy_x) {
    const mrs_m3_config &c = bb->cfg;
    const int ng = c.ngroups, ds = c.d_state;
    const size_t lds = (size_t)(2 * ng * ds + 2 * ng) * sizeof(float);
    if (lds > 60000) return fail(MRS_E_SHAPE, "m3 K/Q kernel: ngroups * d_state too large for LDS (%zu bytes)", lds);
    if (ng == 1 && ds % 4 == 0 && ldbc % 4 == 0 && aligned(bc, 16)) {
        hipLaunchKernelGGL((m3_kq_rows_kernel<T>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, bb->stream, (T *)bb->pf_K, (T *)bb->pf_Q,
                           copy_x ? (T *)bb->pf_x : nullptr, (const T *)bulk, ldb, bc, ldbc, bb->pf_angle, lw.bnw, lw.cnw, lw.b_bias, lw.c_bias, rows,
                           bb->nh, c.headdim, ds, bb->nr, c.rms_norm_eps);
        return check_launch("m3_kq_rows_kernel");
    }
    hipLaunchKernelGGL((m3_kq_kernel<T>), dim3((unsigned)rows), dim3(256), lds, bb->stream, (T *)bb->pf_K, (T *)bb->pf_Q,
                       copy_x ? (T *)bb->pf_x : nullptr, (const T *)bulk, ldb, bc, ldbc, bb->pf_angle, lw.bnw, lw.cnw, lw.b_bias, lw.c_bias, bb->nh,
                       c.headdim, ng, ds, bb->nr, c.rms_norm_eps);
    return check_launch("m3_kq_kernel");
}

template <typename T>
int launch_gate_t(mrs_m3_backbone *bb, const Layer3 &lw, int64_t rows, const void *bulk, int64_t ldb) {
    const mrs_m3_config &c = bb->cfg;
    constexpr int V = 16 / (int)sizeof(T);
    if (!c.is_outproj_norm && bb->di % V == 0 && ldb % V == 0 && aligned(bulk, 16) && rows * (bb->di / V) < 0x7fffffffLL * 256) {
        const int64_t n = (rows + kGateRows - 1) / kGateRows * (bb->di / V);
        hipLaunchKernelGGL((m3_gate_silu_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, bb->stream, (T *)bb->pf_gated,
                           (const T *)bb->pf_y, (const T *)bulk, ldb, rows, bb->di);
        return check_launch("m3_gate_silu_kernel");
    }
    hipLaunchKernelGGL((m3_gate_kernel<T>), dim3((unsigned)rows), dim3(256), 0, bb->stream, (T *)bb->pf_gated, (const T *)bb->pf_y,
                       (const T *)bulk, ldb, lw.ngw, bb->nh, c.headdim, c.rms_norm_eps, c.is_outproj_norm);
    return check_launch("m3_gate_kernel");
}

int launch_add_rmsnorm3(mrs_m3_backbone *bb, float *residual, const void *add, void *out, bool out_f32, const float *w, int64_t rows) {
    return launch_add_rmsnorm_any(bb->stream, bb->dtype, residual, add, out, out_f32, nullptr, w, bb->cfg.rms_norm_eps, rows, bb->cfg.d_model,
                                  bb->cfg.d_model);
}

int prefill_body3(mrs_m3_backbone *bb, int T) {
    const mrs_m3_config &c = bb->cfg;
    const int dm = c.d_model, di = bb->di, B = bb->batch, dt = bb->dtype, L = c.n_layers, ip = bb->ip, nh = bb->nh, hd = c.headdim, ds = c.d_state;
    const int64_t rows = (int64_t)B * T;
    const size_t es = esize3(dt);
    const int nr = bb->nr;
    if (bb->identity_proj) {
        MRS_HIP(hipMemcpyAsync(bb->pf_residual, bb->pf_in, (size_t)rows * dm * 4, hipMemcpyDeviceToDevice, bb->stream));
    } else {
        const int64_t n = rows * dm;
        hipLaunchKernelGGL(bias_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, bb->stream, bb->pf_residual, bb->input_proj_b, n, dm);
        const float one = 1.0f;
        MRS_BLAS(rocblas_gemm_ex(bb->blas, rocblas_operation_none, rocblas_operation_none, dm, (int)rows, bb->input_dim, &one, bb->input_proj_w,
                                 rocblas_datatype_f32_r, dm, bb->pf_in, rocblas_datatype_f32_r, bb->input_dim, &one, bb->pf_residual,
                                 rocblas_datatype_f32_r, dm, bb->pf_residual, rocblas_datatype_f32_r, dm, rocblas_datatype_f32_r,
                                 rocblas_gemm_algo_standard, 0, 0));
    }
    const bool chunked_ok = (hd == 16 || hd == 32 || hd == 64) && (ds == 16 || ds == 32 || ds == 64);
    const bool no_fused_kq = getenv("MRS_M3_NO_FUSED_KQ") != nullptr;   // keeps the separate K / Q pass (measurement, tests)
    for (int l = 0; l < L; l++) {
        const Layer3 &lw = bb->layers[l];
        float *ssm = bb->ssm + (size_t)l * B * nh * hd * ds, *kst = bb->kst + (size_t)l * B * nh * ds;
        float *vst = bb->vst + (size_t)l * B * nh * hd, *ang = bb->angle + (size_t)l * B * nh * (nr > 0 ? nr : 1);
        MRS_TRY(launch_add_rmsnorm3(bb, bb->pf_residual, l == 0 ? nullptr : bb->pf_out, bb->pf_normed, false, lw.norm_w, rows));
        // in_proj.  The bulk columns (z, x) come out in the storage type; B, C, the head scalars and the angle inputs
        // (the last 2 ng ds + 3 nh + nr columns) in f32 whatever the storage type, as the decode step sees them -- two
        // GEMMs over column slices of the same weight for 16-bit storage, one for f32.  (The bulk slice is 2 d_inner wide
        // on purpose: with B and C in it the 768-wide shape's 3200 columns cost the vendor kernel a third more time
        // than 3072 do.)
        const int nb = 2 * di, ns = ip - nb, nbc = 2 * c.ngroups * ds;
        const void *bulk; int64_t ldb; const float *scp, *bcp; int64_t lds_;
        {
            const rocblas_datatype t = blas_type3(dt), f32t = rocblas_datatype_f32_r;
            auto gemm = [&](int ta, int m, const void *W, int ldw, void *C, rocblas_datatype ct, int ldc) {
                return gemm_ex_tuned(bb->tuner, bb->blas, bb->stream, ta, m, (int)rows, dm, W, t, ldw, bb->pf_normed, t, dm, C, ct, ldc);
            };
            if (dt == MRS_F32) {
                MRS_TRY(gemm(0, ip, lw.in_proj, ip, bb->pf_proj, t, ip));
                bulk = bb->pf_proj; ldb = ip; bcp = bb->pf_proj + nb; scp = bcp + nbc; lds_ = ip;
            } else {
                // the vendor kernels for the transposed operand are faster at these shapes (the copy's first nb rows, then the rest)
                if (lw.in_proj_t) {
                    MRS_TRY(gemm(1, nb, lw.in_proj_t, dm, bb->pf_bulk, t, nb));
                    MRS_TRY(gemm(1, ns, (const char *)lw.in_proj_t + (size_t)nb * dm * es, dm, bb->pf_proj, f32t, ns));
                } else {
                    MRS_TRY(gemm(0, nb, lw.in_proj, ip, bb->pf_bulk, t, nb));
                    MRS_TRY(gemm(0, ns, (const char *)lw.in_proj + (size_t)nb * es, ip, bb->pf_proj, f32t, ns));
                }
                bulk = bb->pf_bulk; ldb = nb; bcp = bb->pf_proj; scp = bcp + nbc; lds_ = ns;
            }
        }
        // the chunked kernel reads x (and the gate z) in place out of the bulk rows
        const bool in_place = chunked_ok && dt != MRS_F32 && ldb % 8 == 0 && di % 8 == 0;
        // one group at headdim = d_state = 64 with the rope pairs in fours: the scan builds its K and Q tiles from the
        // normalised B / C rows and the angles, so the [rows, nheads, d_state] K and Q never exist in memory
        const bool fused_kq = in_place && hd == 64 && ds == 64 && c.ngroups == 1 && nr > 0 && nr % 4 == 0 && !no_fused_kq;
        // that scan reads a head's step scalars and angles as runs of steps (a chunk's 64 steps of one head are 256
        // bytes instead of 4 bytes in each of 64 rows): the kernels in front of it write them that way
        const size_t turned_bytes = (size_t)3 * nh * (kScalarRows + 1) * sizeof(float);
        const bool head_major = fused_kq && turned_bytes <= 48 * 1024;
        {
            MRS_DISPATCH_DTYPE(dt, T_, hipLaunchKernelGGL(m3_scalars_kernel<T_>, dim3((unsigned)((rows + kScalarRows - 1) / kScalarRows)), dim3(1024),
                                                          head_major ? turned_bytes : 0, bb->stream, bb->pf_dt, bb->pf_a, bb->pf_trap, bb->pf_tanhpi,
                                                          head_major ? bb->pf_dtT : nullptr, bb->pf_aT, bb->pf_trapT, scp, lds_, lw.dt_bias, rows, T, nh,
                                                          nr, 0, c.a_floor, fused_kq ? (T_ *)bb->pf_bcn : nullptr, bcp, lds_, lw.bnw, lw.cnw,
                                                          c.rms_norm_eps));
            MRS_TRY(check_launch("m3_scalars_kernel"));
        }
        if (nr > 0) {
            const int per = nh * nr, threads = std::min(1024, (per + 63) / 64 * 64);
            const int nsegs = std::max(1, std::min(kAngleSegs, T / 8));
            hipLaunchKernelGGL(m3_angle_sums_kernel, dim3((unsigned)(B * nsegs)), dim3((unsigned)threads), 0, bb->stream, bb->pf_angle_sums,
                               bb->pf_angle_snap, ang, bb->pf_dt, bb->pf_tanhpi, T, nh, nr, nsegs);
            MRS_TRY(check_launch("m3_angle_sums_kernel"));
            hipLaunchKernelGGL(m3_angle_apply_kernel, dim3((unsigned)(B * nsegs)), dim3((unsigned)threads), 0, bb->stream, bb->pf_angle, ang,
                               bb->pf_angle_sums, bb->pf_angle_snap, bb->pf_dt, bb->pf_tanhpi, T, nh, nr, nsegs, head_major ? 1 : 0);
            MRS_TRY(check_launch("m3_angle_apply_kernel"));
        }
        bool gate_in_scan = false;
        if (fused_kq) {
            // the plain SiLU gate rides on the scan's output store (z = the first d_inner elements of the bulk rows): no gate
            // pass, and y itself is never written
            gate_in_scan = !c.is_outproj_norm && ldb % 8 == 0;
            const SsdGenArgs gen = {bb->pf_bcn, (const char *)bb->pf_bcn + (size_t)ds * es, 2 * (int64_t)ds, bb->pf_angle, lw.b_bias, lw.c_bias, nr, head_major ? 1 : 0,
                                    gate_in_scan ? bulk : nullptr, ldb};
            const char *xb = (const char *)bulk + (size_t)di * es;
            MRS_TRY(m3_ssd_fwd_ex(bb->stream, dt, ssm, kst, vst, gate_in_scan ? bb->pf_gated : bb->pf_y, xb, ldb, nullptr, nullptr, head_major ? bb->pf_dtT : bb->pf_dt,
                                  head_major ? bb->pf_trapT : bb->pf_trap, head_major ? bb->pf_aT : bb->pf_a, lw.D,
                                  bb->pf_ws, bb->pf_ws_bytes, MRS_M3_CARRY_STATE, B, T, nh, hd, ds, 64, &gen));
        } else if (in_place) {
            MRS_DISPATCH_DTYPE(dt, T_, MRS_TRY(launch_kq_t<T_>(bb, lw, rows, bulk, ldb, bcp, lds_, false)));
            const char *xb = (const char *)bulk + (size_t)di * es;
            MRS_TRY(m3_ssd_fwd_ex(bb->stream, dt, ssm, kst, vst, bb->pf_y, xb, ldb, bb->pf_K, bb->pf_Q, bb->pf_dt, bb->pf_trap, bb->pf_a, lw.D,
                                  bb->pf_ws, bb->pf_ws_bytes, MRS_M3_CARRY_STATE, B, T, nh, hd, ds, 64));
        } else if (chunked_ok) {
            MRS_DISPATCH_DTYPE(dt, T_, MRS_TRY(launch_kq_t<T_>(bb, lw, rows, bulk, ldb, bcp, lds_, true)));
            MRS_TRY(mrs_m3_ssd_fwd(bb->stream, dt, ssm, kst, vst, bb->pf_y, bb->pf_x, bb->pf_K, bb->pf_Q, bb->pf_dt, bb->pf_trap, bb->pf_a, lw.D,
                                   bb->pf_ws, bb->pf_ws_bytes, MRS_M3_CARRY_STATE, B, T, nh, hd, ds, 64));
        } else {
            MRS_DISPATCH_DTYPE(dt, T_, MRS_TRY(launch_kq_t<T_>(bb, lw, rows, bulk, ldb, bcp, lds_, true)));
            float *al = (float *)bb->pf_ws, *be = al + rows * nh, *ga = be + rows * nh;
            MRS_TRY(mrs_m3_compute_abg(bb->stream, al, be, ga, bb->pf_dt, bb->pf_a, bb->pf_trap, rows * nh));
            MRS_TRY(mrs_m3_seq_fwd(bb->stream, dt, ssm, kst, vst, bb->pf_y, bb->pf_x, bb->pf_K, bb->pf_Q, al, be, ga, lw.D, B, T, nh, hd, ds));
        }
        if (!gate_in_scan) MRS_DISPATCH_DTYPE(dt, T_, MRS_TRY(launch_gate_t<T_>(bb, lw, rows, bulk, ldb)));
        MRS_TRY(gemm3(bb, bb->pf_out, false, bb->pf_gated, lw.out_proj, (int)rows, dm, di));
    }
    // only the last position of each sequence is kept: final residual add + norm_f on those rows
    for (int b = 0; b < B; b++) {
        const size_t r = (size_t)b * T + (T - 1);
        MRS_TRY(launch_add_rmsnorm3(bb, bb->pf_residual + r * dm, (const char *)bb->pf_out + r * dm * es, bb->temporal + (size_t)b * dm, true,
                                    bb->norm_f, 1));
    }
    return MRS_OK;
}

}  // namespace

extern "C" int mrs_m3_backbone_set_gemm_tuning(mrs_m3_backbone *bb, int on) {
    if (!bb) return fail(MRS_E_NULL, "mrs_m3_backbone_set_gemm_tuning: null engine");
    gemm_tuner_enable(bb->tuner, on);
    return MRS_OK;
}

// Runs the sequences already in prefill_input_ptr() ([batch, T, input_dim] f32), continuing from the engine's state and
// leaving it positioned for step(); norm_f output of the last position in temporal_ptr().
extern "C" int mrs_m3_backbone_prefill_device(mrs_m3_backbone *bb, int T) {
    if (!bb) return fail(MRS_E_NULL, "mrs_m3_backbone_prefill_device: null engine");
    if (T < 1) return fail(MRS_E_SHAPE, "mrs_m3_backbone_prefill_device: T=%d", T);
    MRS_TRY(mrs_m3_backbone_alloc_prefill_scratch(bb, T));
    return prefill_body3(bb, T);
}

extern "C" int mrs_m3_backbone_prefill_sequence(mrs_m3_backbone *bb, const float *input, int T, float *out_last) {
    if (!bb || !input) return fail(MRS_E_NULL, "mrs_m3_backbone_prefill_sequence: null pointer");
    if (T < 1) return fail(MRS_E_SHAPE, "mrs_m3_backbone_prefill_sequence: T=%d", T);
    MRS_TRY(mrs_m3_backbone_alloc_prefill_scratch(bb, T));
    MRS_HIP(hipMemcpyAsync(bb->pf_in, input, (size_t)bb->batch * T * bb->input_dim * 4, hipMemcpyHostToDevice, bb->stream));
    MRS_TRY(prefill_body3(bb, T));
    if (out_last) MRS_HIP(hipMemcpyAsync(out_last, bb->temporal, (size_t)bb->batch * bb->cfg.d_model * 4, hipMemcpyDeviceToHost, bb->stream));
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}

extern "C" float *mrs_m3_backbone_prefill_input_ptr(mrs_m3_backbone *bb) { return bb ? bb->pf_in : nullptr; }

extern "C" float *mrs_m3_backbone_temporal_ptr(mrs_m3_backbone *bb) { return bb ? bb->temporal : nullptr; }
extern "C" int mrs_m3_backbone_temporal_dtype(mrs_m3_backbone *bb) { return bb ? MRS_F32 : -1; }
extern "C" int mrs_m3_backbone_decode_route(mrs_m3_backbone *bb) {
    if (!bb) return -1;
    return bb->tiny_layers ? MRS_DECODE_ONE_LAUNCH : bb->skinny ? MRS_DECODE_OWN_CHAIN : MRS_DECODE_LIBRARY_CHAIN;
}
extern "C" float *mrs_m3_backbone_input_ptr(mrs_m3_backbone *bb) { return bb ? bb->d_input : nullptr; }
extern "C" void *mrs_m3_backbone_stream(mrs_m3_backbone *bb) { return bb ? (void *)bb->stream : nullptr; }
extern "C" int mrs_m3_backbone_sync(mrs_m3_backbone *bb) {
    if (!bb) return fail(MRS_E_NULL, "mrs_m3_backbone_sync: null engine");
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}

// Copies layer `layer`'s state to host buffers (any may be null): ssm [batch,nh,hd,ds], k [batch,nh,ds], v [batch,nh,hd],
// angle [batch,nh,max(n_rope,1)].
extern "C" int mrs_m3_backbone_download_state(mrs_m3_backbone *bb, int layer, float *ssm, float *k, float *v, float *angle) {
    if (!bb) return fail(MRS_E_NULL, "mrs_m3_backbone_download_state: null engine");
    if (layer < 0 || layer >= bb->cfg.n_layers) return fail(MRS_E_SHAPE, "mrs_m3_backbone_download_state: layer %d", layer);
    const size_t B = bb->batch, nh = bb->nh, hd = bb->cfg.headdim, ds = bb->cfg.d_state, na = bb->nr > 0 ? bb->nr : 1, l = layer;
    if (ssm) MRS_HIP(hipMemcpyAsync(ssm, bb->ssm + l * B * nh * hd * ds, B * nh * hd * ds * 4, hipMemcpyDeviceToHost, bb->stream));
    if (k) MRS_HIP(hipMemcpyAsync(k, bb->kst + l * B * nh * ds, B * nh * ds * 4, hipMemcpyDeviceToHost, bb->stream));
    if (v) MRS_HIP(hipMemcpyAsync(v, bb->vst + l * B * nh * hd, B * nh * hd * 4, hipMemcpyDeviceToHost, bb->stream));
    if (angle) MRS_HIP(hipMemcpyAsync(angle, bb->angle + l * B * nh * na, B * nh * na * 4, hipMemcpyDeviceToHost, bb->stream));
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}

// ---- the Mamba-3 engine behind the LM loop (GpuMamba3LM, src/module/gpu_lm3.rs:54-400) ---------------------------
namespace {
void m3_state_sizes(mrs_m3_backbone *bb, size_t (&n)[4]) {
    const size_t L = bb->cfg.n_layers, B = bb->batch, nh = bb->nh, hd = bb->cfg.headdim, ds = bb->cfg.d_state, na = bb->nr > 0 ? bb->nr : 1;
    n[0] = L * B * nh * hd * ds * 4; n[1] = L * B * nh * ds * 4; n[2] = L * B * nh * hd * 4; n[3] = L * B * nh * na * 4;
}
int m3_hook_step(void *self) { return step_body3((mrs_m3_backbone *)self); }
int m3_hook_reset(void *self) { return mrs_m3_backbone_reset((mrs_m3_backbone *)self); }
size_t m3_hook_state_bytes(void *self) {
    size_t n[4];
    m3_state_sizes((mrs_m3_backbone *)self, n);
    return n[0] + n[1] + n[2] + n[3];
}
int m3_hook_state_copy(void *self, void *buf, int restore) {
    mrs_m3_backbone *bb = (mrs_m3_backbone *)self;
    size_t n[4];
    m3_state_sizes(bb, n);
    float *parts[4] = {bb->ssm, bb->kst, bb->vst, bb->angle};
    char *p = (char *)buf;
    for (int i = 0; i < 4; i++) {
        if (restore) MRS_HIP(hipMemcpyAsync(parts[i], p, n[i], hipMemcpyDeviceToDevice, bb->stream));
        else MRS_HIP(hipMemcpyAsync(p, parts[i], n[i], hipMemcpyDeviceToDevice, bb->stream));
        p += n[i];
    }
    return MRS_OK;
}
int m3_hook_prefill(void *self, const int *dev_tokens, const void *embed, int vocab, int T) {
    mrs_m3_backbone *bb = (mrs_m3_backbone *)self;
    MRS_TRY(mrs_m3_backbone_alloc_prefill_scratch(bb, T));
    MRS_TRY(launch_embed_gather(bb->stream, bb->dtype, bb->pf_in, embed, dev_tokens, (int64_t)bb->batch * T, bb->cfg.d_model, vocab));
    return prefill_body3(bb, T);
}
}  // namespace

// LM loop (embedding gather, head, greedy pick or sampling, generate / generate_batch) over a Mamba-3 backbone: every
// mrs_lm_* entry point then works on the returned handle.  embed: [vocab, d_model] f32 on the host.
extern "C" int mrs_lm3_create(mrs_lm **out, mrs_m3_backbone *bb, const float *embed, int vocab) {
    if (!out || !bb || !embed) return fail(MRS_E_NULL, "mrs_lm3_create: null pointer");
    LmHooks h = {};
    h.self = bb; h.batch = bb->batch; h.d_model = bb->cfg.d_model; h.dtype = bb->dtype; h.identity_proj = bb->identity_proj;
    h.stream = bb->stream; h.blas = bb->blas; h.d_input = bb->d_input; h.temporal = bb->temporal; h.temporal_t = nullptr;
    h.step = m3_hook_step; h.reset = m3_hook_reset; h.state_bytes = m3_hook_state_bytes; h.state_copy = m3_hook_state_copy;
    h.prefill = m3_hook_prefill;
    return mrs_lm_create_from_hooks(out, h, embed, vocab, "mrs_lm3_create");
}
