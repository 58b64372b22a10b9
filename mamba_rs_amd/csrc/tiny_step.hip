// A whole Mamba-1 backbone step in one launch for small f32 models (d_inner <= 512: the reference's default
// configuration, d_model 128 x 3 layers, and the tiny CPU-runnable one).  The reference runs such a step as 4 GEMMs and
// 10 kernels per layer (GpuMambaBackbone::step, src/mamba_ssm/gpu/inference.rs:993-1252); at this size every one of them
// is a launch that moves a few kilobytes, so a step costs its launch count (3 layers: 21 launches, 50 us in a graph).
// The batch rows of a step never meet, and a row's activations (d_model + 2 d_inner + ... floats) fit in LDS many times
// over, so one workgroup walks one batch row through input projection, every layer and the final norm: products as
// matrix-vector sweeps over weights that sit in L2 (shared by all rows), the layer's conv window and SSM state read and
// written in place.  Arithmetic per element is that of the separate kernels (same softplus, SiLU, exp2 forms, f32
// accumulation); only the order of the dot-product sums differs, and it is fixed (same result on every run).
#include "tiny_rows.hpp"
#include <algorithm>

namespace mrs {
namespace {

__global__ __launch_bounds__(kTinyThreads) void tiny_backbone_step_kernel(TinyStepArgs a) {
    extern __shared__ float lds[];
    const int dm = a.dm, di = a.di, ds = a.ds, dc = a.dc, dr = a.dr, xd = a.xd;
    const int xin_n = rup4(a.input_dim > dm ? a.input_dim : dm), di4 = rup4(di);
    float *res = lds;                   // [dm]      residual stream of this row
    float *xin = res + rup4(dm);        // [max(dm, input_dim)] operand of the product in flight (input row, normed row)
    float *proj = xin + xin_n;          // [2 di]    in_proj output: x half, gate half
    float *u = proj + rup4(2 * di);     // [di]      conv + SiLU output
    float *dl = u + di4;                // [di]      delta
    float *y = dl + di4;                // [di]      gated scan output
    float *xdbl = y + di4;              // [xd]      x_proj output: dt input, B, C
    float *part = xdbl + rup4(xd);      // [kTinyPart]
    float *red = part + kTinyPart;      // [waves]
    const int tid = threadIdx.x, b = blockIdx.x;
    const int lg = ds >> 2, rows_pp = kTinyThreads / lg;   // scan step: ds / 4 lanes per channel, one float4 of state each
    const int g = tid % lg, d0 = tid / lg;

    TinyStepLayer lnext = a.layers[0];
    // input row -> residual stream (identity or projection + bias)
    for (int i = tid; i < a.input_dim; i += kTinyThreads) xin[i] = a.input[(int64_t)b * a.input_dim + i];
    __syncthreads();
    if (a.in_w) {
        gemv_rows(a.in_w, a.input_dim, dm, xin, res, part, a.in_b);
    } else {
        for (int i = tid; i < dm; i += kTinyThreads) res[i] = xin[i];
        __syncthreads();
    }

    for (int l = 0; l < a.n_layers; l++) {
        // this layer's table entry was read a layer ago, the next one's is read now: the pointer fetch is off the critical path
        const TinyStepLayer lw = lnext;
        lnext = a.layers[min(l + 1, a.n_layers - 1)];
        // what the layer needs from memory whatever its input turns out to be is requested ahead of its use: the conv
        // window, taps and bias of channel tid and the norm weight now, the dt weights and the first two passes' float4s
        // of SSM state with their a_neg and D after in_proj
        float *cst = a.conv_state + ((int64_t)l * a.batch + b) * di * dc;
        float *hst = a.ssm_state + ((int64_t)l * a.batch + b) * di * ds;
        float cwin[8], ctap[8], cbias = 0.0f;
        const bool chan = tid < di;
        if (chan) {
            cbias = lw.conv_b[tid];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                cwin[k] = k < dc ? cst[(int64_t)tid * dc + k] : 0.0f;
                ctap[k] = k < dc ? lw.conv_w[(int64_t)tid * dc + k] : 0.0f;
            }
        }
        const float nw = tid < dm ? lw.norm_w[tid] : 0.0f;
        // RMSNorm of the residual stream
        float ss = 0.0f;
        for (int i = tid; i < dm; i += kTinyThreads) ss = fmaf(res[i], res[i], ss);
        const float inv = rms_inv(block_sum(ss, red), dm, a.eps);
        if (tid < dm) xin[tid] = res[tid] * inv * nw;
        for (int i = tid + kTinyThreads; i < dm; i += kTinyThreads) xin[i] = res[i] * inv * lw.norm_w[i];
        __syncthreads();
        gemv_rows(lw.in_proj, dm, 2 * di, xin, proj, part, nullptr);
        float dtb = 0.0f, dtw[8];
        if (chan) {
            dtb = lw.dt_b[tid];
#pragma unroll
            for (int k = 0; k < 8; k++) dtw[k] = lw.dt_w[(int64_t)min(k, dr - 1) * di + tid];
        }
        float4 hvp[kTinyPre], avp[kTinyPre];
        float Dp[kTinyPre];
#pragma unroll
        for (int p = 0; p < kTinyPre; p++) {
            const int d = d0 + p * rows_pp;
            hvp[p] = avp[p] = make_float4(0.f, 0.f, 0.f, 0.f);
            Dp[p] = 0.0f;
            if (d < di) {
                hvp[p] = *reinterpret_cast<const float4 *>(hst + (int64_t)d * ds + 4 * g);
                avp[p] = *reinterpret_cast<const float4 *>(lw.a_neg + (int64_t)d * ds + 4 * g);
                Dp[p] = lw.D[d];
            }
        }
        // conv1d step + SiLU on the x half (window slot k holds the input d_conv - k steps back; the new input goes last)
        if (chan) {
            float s = cbias;
#pragma unroll
            for (int k = 0; k < 8; k++) {
                if (k < dc) {
                    const float v = k + 1 < dc ? cwin[k + 1 < 8 ? k + 1 : 7] : proj[tid];
                    s = fmaf(v, ctap[k], s);
                    cst[(int64_t)tid * dc + k] = v;
                }
            }
            u[tid] = silu(s);
        }
        __syncthreads();
        gemv_rows(lw.x_proj, di, xd, u, xdbl, part, nullptr);
        // dt_proj + bias + softplus
        if (chan) {
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) s = fmaf(j < dr ? xdbl[j] : 0.0f, dtw[j], s);
            for (int r0 = 8; r0 < dr; r0 += 8) {   // dt_rank beyond 8: eight weight loads in flight at a time
                float wv[8];
#pragma unroll
                for (int j = 0; j < 8; j++) wv[j] = lw.dt_w[(int64_t)min(r0 + j, dr - 1) * di + tid];
#pragma unroll
                for (int j = 0; j < 8; j++) s = fmaf(r0 + j < dr ? xdbl[r0 + j] : 0.0f, wv[j], s);
            }
            dl[tid] = softplus20(s + dtb);
        }
        __syncthreads();
        // scan step + D skip + SiLU gate (the arithmetic of ssm_step_kernel)
        for (int d = d0, pass = 0; d < di; d += rows_pp, pass++) {
            float4 hv, av;
            float Dd;
            if (pass == 0) { hv = hvp[0]; av = avp[0]; Dd = Dp[0]; }
            else if (pass == 1) { hv = hvp[kTinyPre - 1]; av = avp[kTinyPre - 1]; Dd = Dp[kTinyPre - 1]; }
            else {
                hv = *reinterpret_cast<const float4 *>(hst + (int64_t)d * ds + 4 * g);
                av = *reinterpret_cast<const float4 *>(lw.a_neg + (int64_t)d * ds + 4 * g);
                Dd = lw.D[d];
            }
            const float *Bv = xdbl + dr + 4 * g, *Cv = xdbl + dr + ds + 4 * g;
            const float du = dl[d] * u[d], x = dl[d] * kLog2e;
            hv.x = fmaf(fast_exp2(x * av.x), hv.x, du * Bv[0]);
            hv.y = fmaf(fast_exp2(x * av.y), hv.y, du * Bv[1]);
            hv.z = fmaf(fast_exp2(x * av.z), hv.z, du * Bv[2]);
            hv.w = fmaf(fast_exp2(x * av.w), hv.w, du * Bv[3]);
            *reinterpret_cast<float4 *>(hst + (int64_t)d * ds + 4 * g) = hv;
            float acc = hv.x * Cv[0];
            acc = fmaf(hv.y, Cv[1], acc);
            acc = fmaf(hv.z, Cv[2], acc);
            acc = fmaf(hv.w, Cv[3], acc);
            for (int m = 1; m < lg; m <<= 1) acc += __shfl_xor(acc, m, kWave);
            if (g == 0) y[d] = fmaf(Dd, u[d], acc) * silu(proj[di + d]);
        }
        __syncthreads();
        gemv_rows(lw.out_proj, di, dm, y, xin, part, nullptr);
        for (int i = tid; i < dm; i += kTinyThreads) res[i] += xin[i];
        __syncthreads();
    }
    float ss = 0.0f;
    for (int i = tid; i < dm; i += kTinyThreads) ss = fmaf(res[i], res[i], ss);
    const float inv = rms_inv(block_sum(ss, red), dm, a.eps);
    for (int i = tid; i < dm; i += kTinyThreads) a.temporal[(int64_t)b * dm + i] = res[i] * inv * a.norm_f[i];
}

size_t tiny_lds_bytes(const TinyStepArgs &a) {
    const int xin_n = rup4(a.input_dim > a.dm ? a.input_dim : a.dm);
    return sizeof(float) * ((size_t)rup4(a.dm) + xin_n + rup4(2 * a.di) + 3 * (size_t)rup4(a.di) + rup4(a.xd) + kTinyPart + kTinyThreads / 64);
}

}  // namespace

bool tiny_step_ok(int dtype, int input_dim, int dm, int di, int ds, int dc, int dr, int xd) {
    if (input_dim < 1 || dm < 4 || di < 2 || xd < 4) return false;
    if (sweep_rounds(input_dim, dm) > kTinyMaxRounds || sweep_rounds(dm, 2 * di) > kTinyMaxRounds || sweep_rounds(di, xd) > kTinyMaxRounds ||
        sweep_rounds(di, dm) > kTinyMaxRounds)
        return false;
    return dtype == MRS_F32 && dm >= 4 && dm % 4 == 0 && dm <= 1024 && di % 4 == 0 && di >= 4 && di <= 512 && xd % 4 == 0 && xd >= 4 &&
           xd <= 1024 && (ds == 4 || ds == 8 || ds == 16 || ds == 32 || ds == 64) && dc >= 1 && dc <= 8 && dr >= 1 && input_dim >= 1 &&
           input_dim <= 4096 && xd == dr + 2 * ds;
}

int launch_tiny_step(hipStream_t st, const TinyStepArgs &a) {
    if (!tiny_step_ok(MRS_F32, a.input_dim, a.dm, a.di, a.ds, a.dc, a.dr, a.xd) || a.batch < 1 || a.n_layers < 1 || !a.layers || !a.input ||
        !a.conv_state || !a.ssm_state || !a.temporal || !a.norm_f)
        return fail(MRS_E_SHAPE, "tiny backbone step: shape outside the single-launch route (d_model=%d d_inner=%d d_state=%d xdbl=%d)", a.dm, a.di,
                    a.ds, a.xd);
    const size_t lds = tiny_lds_bytes(a);
    if (lds > 64 * 1024) return fail(MRS_E_SHAPE, "tiny backbone step: %zu bytes of LDS", lds);
    hipLaunchKernelGGL(tiny_backbone_step_kernel, dim3((unsigned)a.batch), dim3(kTinyThreads), lds, st, a);
    return check_launch("tiny_backbone_step_kernel");
}

}  // namespace mrs
