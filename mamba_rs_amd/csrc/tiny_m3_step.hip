// A whole Mamba-3 SISO backbone step in one launch for small f32 models (the reference's default configuration:
// d_model 128, 4 layers, headdim 16, d_state 16).  GpuMamba3Backbone::step runs such a step as fourteen launches per
// layer (src/mamba3_siso/gpu/inference.rs:506-1000), the engine here as three; at this size each of them moves a few
// kilobytes and costs its launch.  One workgroup walks one batch row through input projection, every layer and the final
// norm: in_proj and out_proj as matrix-vector sweeps over weights that sit in L2, the layer step between them with the
// formulas of m3_layer_step_kernel (B/C RMSNorm + bias, angle accumulation in f64 and rotation, alpha / beta / gamma,
// the trapezoidal state update, D skip, SiLU gate or RMSNormGated), states updated in place.  Only the order of the
// dot-product sums differs from the kernel chain, and it is fixed.
#include "tiny_rows.hpp"
#include "m3_math.hpp"

namespace mrs {
namespace {

__global__ __launch_bounds__(kTinyThreads) void tiny_m3_backbone_step_kernel(TinyM3StepArgs a) {
    extern __shared__ float lds[];
    const int dm = a.dm, di = a.di, nh = a.nh, hd = a.hd, ds = a.ds, ng = a.ng, nr = a.nr, ip = a.ip;
    const int xin_n = rup4(a.input_dim > dm ? a.input_dim : dm), di4 = rup4(di);
    float *res = lds;                   // [dm]       residual stream of this row
    float *xin = res + rup4(dm);        // [max(dm, input_dim)] operand of the product in flight
    float *proj = xin + xin_n;          // [ip]       in_proj output: z | x | B | C | dd_dt | dd_A | trap | angles
    float *kl = proj + rup4(ip);        // [nh ds]    K of every head (normalised, biased, rotated B)
    float *ql = kl + rup4(nh * ds);     // [nh ds]    Q of every head
    float *yr = ql + rup4(nh * ds);     // [di]       y before the gate
    float *yg = yr + di4;               // [di]       gated y: out_proj's operand
    float *ginv = yg + di4;             // [2 ng]     1 / rms of the raw B and C rows per group
    float *part = ginv + rup4(2 * ng);  // [kTinyPart]
    float *red = part + kTinyPart;      // [waves]
    const int tid = threadIdx.x, b = blockIdx.x;
    const int lg = ds >> 2, per_head = hd * lg, tasks = nh * per_head;   // one lane-task per float4 of SSM state
    const int na = nr > 0 ? nr : 1;

    for (int i = tid; i < a.input_dim; i += kTinyThreads) xin[i] = a.input[(int64_t)b * a.input_dim + i];
    __syncthreads();
    if (a.in_w) {
        gemv_rows(a.in_w, a.input_dim, dm, xin, res, part, a.in_b);
    } else {
        for (int i = tid; i < dm; i += kTinyThreads) res[i] = xin[i];
        __syncthreads();
    }

    TinyM3StepLayer lnext = a.layers[0];
    for (int l = 0; l < a.n_layers; l++) {
        const TinyM3StepLayer lw = lnext;
        lnext = a.layers[min(l + 1, a.n_layers - 1)];
        float *ssm = a.ssm + ((int64_t)l * a.batch + b) * nh * hd * ds;
        float *kst = a.kst + ((int64_t)l * a.batch + b) * nh * ds;
        float *vst = a.vst + ((int64_t)l * a.batch + b) * nh * hd;
        float *ang = a.angle + ((int64_t)l * a.batch + b) * nh * na;
        // RMSNorm of the residual stream, in_proj
        float ss = 0.0f;
        for (int i = tid; i < dm; i += kTinyThreads) ss = fmaf(res[i], res[i], ss);
        const float inv = rms_inv(block_sum(ss, red), dm, a.eps);
        for (int i = tid; i < dm; i += kTinyThreads) xin[i] = res[i] * inv * lw.norm_w[i];
        __syncthreads();
        gemv_rows(lw.in_proj, dm, ip, xin, proj, part, nullptr);
        const float *braw = proj + 2 * di, *craw = braw + ng * ds;
        const float *sc = proj + 2 * di + 2 * ng * ds;   // dd_dt | dd_A | trap | angles
        // B/C RMSNorm over d_state per group (bcnorm_fwd, ops/norms.rs:50-80)
        for (int grp = 0; grp < ng; grp++) {
            float sb = 0.0f, scs = 0.0f;
            for (int n = tid; n < ds; n += kTinyThreads) {
                sb = fmaf(braw[grp * ds + n], braw[grp * ds + n], sb);
                scs = fmaf(craw[grp * ds + n], craw[grp * ds + n], scs);
            }
            sb = block_sum(sb, red);
            scs = block_sum(scs, red);
            if (tid == 0) {
                ginv[2 * grp] = 1.0f / sqrtf(sb / (float)ds + a.eps);
                ginv[2 * grp + 1] = 1.0f / sqrtf(scs / (float)ds + a.eps);
            }
        }
        __syncthreads();
        // K and Q of every head: weight, per-head bias
        for (int i = tid; i < nh * ds; i += kTinyThreads) {
            const int h = i / ds, n = i - h * ds, grp = h / (nh / ng);
            kl[i] = braw[grp * ds + n] * ginv[2 * grp] * lw.bnw[n] + lw.b_bias[i];
            ql[i] = craw[grp * ds + n] * ginv[2 * grp + 1] * lw.cnw[n] + lw.c_bias[i];
        }
        __syncthreads();
        // angle accumulation (f64, wrapped to [0, 2 pi)) and rotation of the first 2 nr coordinates of K and Q
        for (int i = tid; i < nh * nr; i += kTinyThreads) {
            const int h = i / nr, r = i - h * nr;
            const float dtv = softplus20(sc[h] + lw.dt_bias[h]);
            const float delta = tanhf(sc[3 * nh + r]) * kPi * dtv;
            const float an = (float)wrap_2pi((double)ang[i] + (double)delta);
            ang[i] = an;
            float sn, cs;
            sincosf(an, &sn, &cs);
            float *kp2 = kl + h * ds + 2 * r, *qp2 = ql + h * ds + 2 * r;
            const float b0 = kp2[0], b1 = kp2[1], c0 = qp2[0], c1 = qp2[1];
            kp2[0] = cs * b0 - sn * b1; kp2[1] = sn * b0 + cs * b1;
            qp2[0] = cs * c0 - sn * c1; qp2[1] = sn * c0 + cs * c1;
        }
        __syncthreads();
        // trapezoidal update of one float4 of state per lane-task, y = H q + D x (lane-task = (head, row p, quad g))
        for (int t = tid; t < tasks; t += kTinyThreads) {
            const int h = t / per_head, rem = t - h * per_head, p = rem / lg, g = rem - p * lg;
            float *Hrow = ssm + ((int64_t)h * hd + p) * ds + 4 * g;
            float4 H = *reinterpret_cast<const float4 *>(Hrow);
            const float4 kp = *reinterpret_cast<const float4 *>(kst + h * ds + 4 * g);
            const float vp = vst[h * hd + p];
            const float xv = proj[di + h * hd + p];
            const float dtv = softplus20(sc[h] + lw.dt_bias[h]);
            const float a_val = fminf(-heavy_tail(sc[nh + h]), -a.a_floor);
            const float trap = sigmoidf_fast(sc[2 * nh + h]);
            const float al = fast_exp2(a_val * dtv * kLog2e);
            const float be = al * dtv * (1.0f - trap), ga = trap * dtv;
            const float4 kc = *reinterpret_cast<const float4 *>(&kl[h * ds + 4 * g]);
            const float4 qc = *reinterpret_cast<const float4 *>(&ql[h * ds + 4 * g]);
            const float bv = be * vp, gx = ga * xv;
            H.x = fmaf(al, H.x, fmaf(bv, kp.x, gx * kc.x));
            H.y = fmaf(al, H.y, fmaf(bv, kp.y, gx * kc.y));
            H.z = fmaf(al, H.z, fmaf(bv, kp.z, gx * kc.z));
            H.w = fmaf(al, H.w, fmaf(bv, kp.w, gx * kc.w));
            float acc = H.x * qc.x;
            acc = fmaf(H.y, qc.y, acc);
            acc = fmaf(H.z, qc.z, acc);
            acc = fmaf(H.w, qc.w, acc);
            for (int m = 1; m < lg; m <<= 1) acc += __shfl_xor(acc, m, kWave);
            *reinterpret_cast<float4 *>(Hrow) = H;
            if (g == 0) yr[h * hd + p] = fmaf(lw.D[h], xv, acc);
        }
        __syncthreads();   // every read of the previous k_state and v_state has returned
        for (int i = tid; i < nh * ds; i += kTinyThreads) kst[i] = kl[i];
        // gate: y * silu(z), or RMSNormGated over the head first (rmsnorm_gated_forward, ops/norms.rs:84-114)
        for (int i = tid; i < di; i += kTinyThreads) {
            const float xv = proj[di + i], zi = proj[i];
            vst[i] = xv;
            float o = yr[i] * silu(zi);
            if (a.outproj_norm) {
                const int h = i / hd;
                float sq = 0.0f;
                for (int p = 0; p < hd; p++) sq = fmaf(yr[h * hd + p], yr[h * hd + p], sq);
                o = yr[i] * (1.0f / sqrtf(sq / (float)hd + a.eps)) * lw.ngw[i] * silu(zi);
            }
            yg[i] = o;
        }
        __syncthreads();
        gemv_rows(lw.out_proj, di, dm, yg, xin, part, nullptr);
        for (int i = tid; i < dm; i += kTinyThreads) res[i] += xin[i];
        __syncthreads();
    }
    float ss = 0.0f;
    for (int i = tid; i < dm; i += kTinyThreads) ss = fmaf(res[i], res[i], ss);
    const float inv = rms_inv(block_sum(ss, red), dm, a.eps);
    for (int i = tid; i < dm; i += kTinyThreads) a.temporal[(int64_t)b * dm + i] = res[i] * inv * a.norm_f[i];
}

size_t tiny_m3_lds_bytes(int input_dim, int dm, int di, int nh, int ds, int ng, int ip) {
    const int xin_n = rup4(input_dim > dm ? input_dim : dm);
    return sizeof(float) * ((size_t)rup4(dm) + xin_n + rup4(ip) + 2 * (size_t)rup4(nh * ds) + 2 * (size_t)rup4(di) + rup4(2 * ng) + kTinyPart + kTinyThreads / 64);
}

}  // namespace

bool tiny_m3_step_ok(int dtype, int input_dim, int dm, int di, int nh, int hd, int ds, int ng, int nr, int ip) {
    if (dtype != MRS_F32 || input_dim < 1 || input_dim > 4096 || dm < 4 || dm % 4 != 0 || dm > 2048 || ip % 4 != 0 || ip > 2048 || di < 1 || di > 1024)
        return false;
    const int lg = ds / 4;
    if (ds % 4 != 0 || lg < 1 || lg > 64 || (lg & (lg - 1)) != 0 || nh < 1 || ng < 1 || nh % ng != 0 || nh * hd != di || nr < 0 || 2 * nr > ds) return false;
    if (ip != 2 * di + 2 * ng * ds + 3 * nh + nr) return false;
    if (sweep_rounds(input_dim, dm) > kTinyMaxRounds || sweep_rounds(dm, ip) > kTinyMaxRounds || sweep_rounds(di, dm) > kTinyMaxRounds) return false;
    return tiny_m3_lds_bytes(input_dim, dm, di, nh, ds, ng, ip) <= 64 * 1024;
}

int launch_tiny_m3_step(hipStream_t st, const TinyM3StepArgs &a) {
    if (!tiny_m3_step_ok(MRS_F32, a.input_dim, a.dm, a.di, a.nh, a.hd, a.ds, a.ng, a.nr, a.ip) || a.batch < 1 || a.n_layers < 1 || !a.layers ||
        !a.input || !a.ssm || !a.kst || !a.vst || !a.angle || !a.temporal || !a.norm_f)
        return fail(MRS_E_SHAPE, "tiny Mamba-3 backbone step: shape outside the single-launch route (d_model=%d d_inner=%d d_state=%d in_proj width=%d)",
                    a.dm, a.di, a.ds, a.ip);
    const size_t lds = tiny_m3_lds_bytes(a.input_dim, a.dm, a.di, a.nh, a.ds, a.ng, a.ip);
    hipLaunchKernelGGL(tiny_m3_backbone_step_kernel, dim3((unsigned)a.batch), dim3(kTinyThreads), lds, st, a);
    return check_launch("tiny_m3_backbone_step_kernel");
}

}  // namespace mrs
