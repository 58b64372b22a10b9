/*
 * m3_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE (see mamba_oracle.c).
 *
 * CPU restatement of the Mamba-3 SISO part of the hot path of silvermpx/mamba-rs
 * v0.5.3: the trapezoidal recurrence (sequential definition), the chunked SSD
 * algebra of kernels/mamba3_chunked.cu, and the per-layer step of
 * src/mamba3_siso/cpu/inference.rs that defines where alpha/beta/gamma, K and Q
 * come from.  Pins live in tests/test_oracle_m3.py:
 *   - sequential recurrence: closed forms (trap = 1 reduces to h = a h + dt x k^T,
 *     alpha = 1 and beta = 0 gives a running sum), independent numpy brute force;
 *   - chunked form: chunked == sequential for every chunk size incl. a partial last
 *     chunk (tests/m3_chunked_fwd_unit_parity.rs shapes), with and without carried state;
 *   - layer step: independent float64 numpy statement of the equations; angle in
 *     [0, 2pi), rotation norm-preserving, reset reproduces, batch == sequential
 *     (src/mamba3_siso/cpu/inference.rs:367-617).
 *
 *   parity unpinned: the carried-state extension of the chunked form (entering
 *   ssm/k/v state folded into chunk 0) has no counterpart in the reference, whose
 *   chunked window is stateless (kernels/mamba3_chunked.cu:219-223); it is pinned
 *   only against the sequential definition, not against reference behaviour.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

float orc_fast_exp(float x);
float orc_round_bf16(float x);
float orc_round_f16(float x);

static inline float round_store(float x, int dtype) {
    if (dtype == 2) return orc_round_bf16(x);
    if (dtype == 1) return orc_round_f16(x);
    return x;
}

/* heavy_tail / softplus, src/mamba3_siso/cpu/forward.rs:146-166 */
static inline float heavy_tail(float x) { return (x >= 0.0f) ? 1.0f + x : 1.0f / (1.0f - x); }
static inline float softplus_cpu(float x) { return (x > 20.0f) ? x : log1pf(orc_fast_exp(x)); }

/* alpha = exp(a dt), beta = alpha dt (1 - trap), gamma = trap dt
 * (m3_compute_abg, kernels/mamba3_ops.cu:735-753; cpu/inference.rs:199-202) in f64. */
ORC_API void orc_m3_abg_f64(double *alpha, double *beta, double *gamma, const float *dt,
                            const float *a_val, const float *trap, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        double al = exp((double)a_val[i] * (double)dt[i]);
        alpha[i] = al;
        beta[i] = al * (double)dt[i] * (1.0 - (double)trap[i]);
        gamma[i] = (double)trap[i] * (double)dt[i];
    }
}

/* -------------------------------------------------------------------------
 * Sequential trapezoidal recurrence over T steps, f64 ground truth
 *   (m3_burnin_fwd_nosave, kernels/mamba3_ssd.cu:453-546; T = 1 is m3_step_fwd :56-215;
 *    CPU: simd_ssm_recurrence, src/mamba3_siso/cpu/forward.rs:85-138)
 *   H[p,n] = alpha H[p,n] + beta v_prev[p] k_prev[n] + gamma x[p] k[n]
 *   y[p]   = sum_n H[p,n] q[n] + D[h] x[p];  then k_prev <- k, v_prev <- x
 * Layouts: ssm [B,nh,hd,ds], kst [B,nh,ds], vst [B,nh,hd]; x,y [B,T,nh*hd];
 *          k,q [B,T,nh,ds]; alpha,beta,gamma [B,T,nh]; D [nh].
 * ------------------------------------------------------------------------- */
ORC_API void orc_m3_seq_f64(double *ssm, double *kst, double *vst, double *y, const float *x,
                            const float *k, const float *q, const double *alpha, const double *beta,
                            const double *gamma, const float *D, int64_t B, int64_t T, int64_t nh,
                            int64_t hd, int64_t ds) {
    int64_t di = nh * hd;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < nh; h++) {
            double *kp = kst + (b * nh + h) * ds;
            double *vp = vst + (b * nh + h) * hd;
            for (int64_t t = 0; t < T; t++) {
                int64_t bt = b * T + t;
                double al = alpha[bt * nh + h], be = beta[bt * nh + h], ga = gamma[bt * nh + h];
                const float *kc = k + (bt * nh + h) * ds;
                const float *qc = q + (bt * nh + h) * ds;
                for (int64_t p = 0; p < hd; p++) {
                    double xv = x[bt * di + h * hd + p];
                    double *H = ssm + ((b * nh + h) * hd + p) * ds;
                    double acc = 0.0;
                    for (int64_t n = 0; n < ds; n++) {
                        H[n] = al * H[n] + be * vp[p] * kp[n] + ga * xv * (double)kc[n];
                        acc += H[n] * (double)qc[n];
                    }
                    y[bt * di + h * hd + p] = acc + (double)D[h] * xv;
                }
                for (int64_t n = 0; n < ds; n++) kp[n] = kc[n];
                for (int64_t p = 0; p < hd; p++) vp[p] = x[bt * di + h * hd + p];
            }
        }
}

/* GPU route in f32 (kernels/mamba3_ssd.cu:453-546 operation order), y rounded to storage. */
ORC_API void orc_m3_seq_gpu(float *ssm, float *kst, float *vst, float *y, const float *x,
                            const float *k, const float *q, const float *alpha, const float *beta,
                            const float *gamma, const float *D, int64_t B, int64_t T, int64_t nh,
                            int64_t hd, int64_t ds, int dtype) {
    int64_t di = nh * hd;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < nh; h++) {
            float *kp = kst + (b * nh + h) * ds;
            float *vp = vst + (b * nh + h) * hd;
            for (int64_t t = 0; t < T; t++) {
                int64_t bt = b * T + t;
                float al = alpha[bt * nh + h], be = beta[bt * nh + h], ga = gamma[bt * nh + h];
                const float *kc = k + (bt * nh + h) * ds;
                const float *qc = q + (bt * nh + h) * ds;
                for (int64_t p = 0; p < hd; p++) {
                    float xv = x[bt * di + h * hd + p];
                    float *H = ssm + ((b * nh + h) * hd + p) * ds;
                    float acc = D[h] * xv;
                    for (int64_t n = 0; n < ds; n++) {
                        H[n] = al * H[n] + be * vp[p] * kp[n] + ga * xv * kc[n];
                        acc += H[n] * qc[n];
                    }
                    y[bt * di + h * hd + p] = round_store(acc, dtype);
                }
                for (int64_t n = 0; n < ds; n++) kp[n] = kc[n];
                for (int64_t p = 0; p < hd; p++) vp[p] = x[bt * di + h * hd + p];
            }
        }
}

/* -------------------------------------------------------------------------
 * Chunked SSD form in f64, kernel by kernel (kernels/mamba3_chunked.cu):
 *   preprocess  :57-115   gamma = dt trap; sgamma_t = dt_{t+1}(1-trap_{t+1}) (0 at T-1);
 *                         scale = sgamma + gamma; K_scaled = K scale; qk_dot = (Q.K) gamma
 *   dA_cumsum   :128-151  inclusive cumsum of a dt inside each chunk
 *   chunk_state :167-209  S_c[p,n] = sum_t exp(dA_end - dA_t) K_scaled[t,n] x[t,p]
 *   state_pass  :232-270  exclusive scan over chunks, state <- exp(dA_end) state + S_c
 *   chunk_scan  :346-419  y_t = exp(dA_t) Q_t.S_enter + sum_{s<t} exp(dA_t-dA_s)(Q_t.K_scaled_s) x_s
 *                               + (D + qk_dot_t) x_t
 *   writeback   :289-330  ssm <- final state, k_state <- K[T-1], v_state <- x[T-1]
 * carry != 0 is this build's extension: chunk 0 enters with
 *   ssm_in + dt_0 (1 - trap_0) v_in (x) k_in   instead of zero (see header).
 * ------------------------------------------------------------------------- */
ORC_API void orc_m3_chunked_f64(double *ssm, double *kst, double *vst, double *y, const float *x,
                                const float *K, const float *Q, const float *dt, const float *trap,
                                const float *a_val, const float *D, int64_t B, int64_t T, int64_t nh,
                                int64_t hd, int64_t ds, int64_t cs, int carry) {
    int64_t di = nh * hd, nc = (T + cs - 1) / cs;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < B; b++)
        for (int64_t h = 0; h < nh; h++) {
            double *scale = (double *)malloc(sizeof(double) * T);
            double *qkdot = (double *)malloc(sizeof(double) * T);
            double *dA = (double *)malloc(sizeof(double) * T);
            double *state = (double *)calloc((size_t)(hd * ds), sizeof(double));
            double *Sc = (double *)malloc(sizeof(double) * hd * ds);
            for (int64_t t = 0; t < T; t++) {
                int64_t i = (b * T + t) * nh + h;
                double g = (double)dt[i] * (double)trap[i];
                double sg = 0.0;
                if (t + 1 < T) {
                    int64_t j = (b * T + t + 1) * nh + h;
                    sg = (double)dt[j] * (1.0 - (double)trap[j]);
                }
                scale[t] = sg + g;
                double dot = 0.0;
                for (int64_t n = 0; n < ds; n++)
                    dot += (double)Q[i * ds + n] * (double)K[i * ds + n];
                qkdot[t] = dot * g;
            }
            for (int64_t c = 0; c < nc; c++) {
                double cum = 0.0;
                for (int64_t t = c * cs; t < T && t < (c + 1) * cs; t++) {
                    int64_t i = (b * T + t) * nh + h;
                    cum += (double)a_val[i] * (double)dt[i];
                    dA[t] = cum;
                }
            }
            if (carry) {
                int64_t i0 = (b * T) * nh + h;
                double sgm1 = (double)dt[i0] * (1.0 - (double)trap[i0]);
                for (int64_t p = 0; p < hd; p++)
                    for (int64_t n = 0; n < ds; n++)
                        state[p * ds + n] = ssm[((b * nh + h) * hd + p) * ds + n] +
                                            sgm1 * vst[(b * nh + h) * hd + p] * kst[(b * nh + h) * ds + n];
            }
            for (int64_t c = 0; c < nc; c++) {
                int64_t t0 = c * cs, t1 = (t0 + cs < T) ? t0 + cs : T;
                double dA_end = dA[t1 - 1];
                /* chunk_scan with the entering state */
                for (int64_t t = t0; t < t1; t++) {
                    int64_t it = (b * T + t) * nh + h;
                    for (int64_t p = 0; p < hd; p++) {
                        double yoff = 0.0;
                        for (int64_t n = 0; n < ds; n++) yoff += (double)Q[it * ds + n] * state[p * ds + n];
                        yoff *= exp(dA[t]);
                        double ydiag = 0.0;
                        for (int64_t s = t0; s < t; s++) {
                            int64_t is = (b * T + s) * nh + h;
                            double qk = 0.0;
                            for (int64_t n = 0; n < ds; n++)
                                qk += (double)Q[it * ds + n] * ((double)K[is * ds + n] * scale[s]);
                            ydiag += exp(dA[t] - dA[s]) * qk * (double)x[(b * T + s) * di + h * hd + p];
                        }
                        double xt = x[(b * T + t) * di + h * hd + p];
                        y[(b * T + t) * di + h * hd + p] = ydiag + yoff + ((double)D[h] + qkdot[t]) * xt;
                    }
                }
                /* chunk_state, then state passing */
                for (int64_t p = 0; p < hd; p++)
                    for (int64_t n = 0; n < ds; n++) {
                        double acc = 0.0;
                        for (int64_t t = t0; t < t1; t++) {
                            int64_t it = (b * T + t) * nh + h;
                            acc += exp(dA_end - dA[t]) * ((double)K[it * ds + n] * scale[t]) *
                                   (double)x[(b * T + t) * di + h * hd + p];
                        }
                        Sc[p * ds + n] = acc;
                    }
                double dec = exp(dA_end);
                for (int64_t i = 0; i < hd * ds; i++) state[i] = dec * state[i] + Sc[i];
            }
            for (int64_t p = 0; p < hd; p++) {
                for (int64_t n = 0; n < ds; n++)
                    ssm[((b * nh + h) * hd + p) * ds + n] = state[p * ds + n];
                vst[(b * nh + h) * hd + p] = x[(b * T + T - 1) * di + h * hd + p];
            }
            for (int64_t n = 0; n < ds; n++) kst[(b * nh + h) * ds + n] = K[((b * T + T - 1) * nh + h) * ds + n];
            free(scale); free(qkdot); free(dA); free(state); free(Sc);
        }
}

/* -------------------------------------------------------------------------
 * Mamba3Weights::init, src/mamba3_siso/weights.rs:51-147 (xorshift64 13,7,17)
 * Flat block: input_proj_w[input_dim,dm] input_proj_b[dm], then per layer
 *   norm_w[dm] in_proj[dm,ip] dt_bias[nh] b_norm_w[ds] c_norm_w[ds] b_bias[nh,ds]
 *   c_bias[nh,ds] D[nh] norm_gate_w[di] out_proj[di,dm];  then norm_f[dm].
 * ------------------------------------------------------------------------- */
typedef struct { uint64_t s; } xs_t;
static inline float xs_f32(xs_t *r) {
    r->s ^= r->s << 13; r->s ^= r->s >> 7; r->s ^= r->s << 17;
    return (float)(r->s & 0xFFFFFF) / 16777216.0f;
}
static void kaiming3(float *w, int64_t n, int64_t fan_in, xs_t *r) {
    float bound = (float)sqrt(3.0 / (double)fan_in);
    for (int64_t i = 0; i < n; i++) w[i] = (xs_f32(r) * 2.0f - 1.0f) * bound;
}

typedef struct { int64_t dm, ds, expand, hd, ng, n_layers, n_rope; float a_floor; int outproj_norm; } m3cfg_t;

static int64_t m3_ip(const m3cfg_t *c) {
    int64_t di = c->dm * c->expand, nh = di / c->hd;
    return 2 * di + 2 * c->ng * c->ds + 3 * nh + c->n_rope;
}
static int64_t m3_layer_count(const m3cfg_t *c) {
    int64_t di = c->dm * c->expand, nh = di / c->hd;
    return c->dm + c->dm * m3_ip(c) + nh + 2 * c->ds + 2 * nh * c->ds + nh + di + di * c->dm;
}
ORC_API int64_t orc_m3_param_count(int64_t dm, int64_t ds, int64_t expand, int64_t hd, int64_t ng,
                                   int64_t n_layers, int64_t n_rope, int64_t input_dim) {
    m3cfg_t c = { dm, ds, expand, hd, ng, n_layers, n_rope, 0.0f, 0 };
    return input_dim * dm + dm + n_layers * m3_layer_count(&c) + dm;
}
ORC_API void orc_m3_weights_init(float *p, int64_t dm, int64_t ds, int64_t expand, int64_t hd, int64_t ng,
                                 int64_t n_layers, int64_t n_rope, int64_t input_dim, uint64_t seed) {
    m3cfg_t c = { dm, ds, expand, hd, ng, n_layers, n_rope, 0.0f, 0 };
    int64_t di = dm * expand, nh = di / hd, ip = m3_ip(&c);
    xs_t rng = { seed ? seed : 1 };                                       /* weights.rs:54 seed.max(1) */
    kaiming3(p, input_dim * dm, input_dim, &rng); p += input_dim * dm;    /* :127 */
    for (int64_t i = 0; i < dm; i++) p[i] = 0.0f; p += dm;
    for (int64_t l = 0; l < n_layers; l++) {
        for (int64_t i = 0; i < dm; i++) p[i] = 1.0f; p += dm;
        float *inw = p; p += dm * ip;
        float *dtb = p; p += nh;
        for (int64_t i = 0; i < 2 * ds; i++) p[i] = 1.0f; p += 2 * ds;    /* b_norm, c_norm = 1 */
        for (int64_t i = 0; i < 2 * nh * ds; i++) p[i] = 1.0f; p += 2 * nh * ds; /* B/C bias = 1 :97-104 */
        for (int64_t i = 0; i < nh; i++) p[i] = 1.0f; p += nh;            /* D = 1 */
        for (int64_t i = 0; i < di; i++) p[i] = 1.0f; p += di;            /* norm_gate = 1 */
        float *outw = p; p += di * dm;
        kaiming3(inw, dm * ip, dm, &rng);                                  /* :130 */
        kaiming3(outw, di * dm, di, &rng);                                 /* :131 */
        float lmin = logf(0.001f), lmax = logf(0.1f);                      /* :134-139 */
        for (int64_t i = 0; i < nh; i++) {
            float dtv = expf(xs_f32(&rng) * (lmax - lmin) + lmin);
            dtb[i] = (dtv > 20.0f) ? dtv : logf(expf(dtv) - 1.0f);
        }
    }
    for (int64_t i = 0; i < dm; i++) p[i] = 1.0f;
}

/* -------------------------------------------------------------------------
 * One Mamba-3 layer, one token, CPU route (src/mamba3_siso/cpu/inference.rs:68-258).
 * State: ssm [nh,hd,ds], kst [nh,ds], vst [nh,hd], angle [nh,max(n_rope,1)].
 * If `taps` is non-NULL it receives, per head, the scan-level quantities the GPU
 * kernels consume: alpha,beta,gamma,dt,trap,a_val [nh] each (6*nh), then k [nh,ds], q [nh,ds].
 * ------------------------------------------------------------------------- */
static void gemv_rm(float *y, const float *x, const float *w, int64_t n_in, int64_t n_out) {
    for (int64_t j = 0; j < n_out; j++) y[j] = 0.0f;
    for (int64_t k = 0; k < n_in; k++) {
        float xv = x[k];
        for (int64_t j = 0; j < n_out; j++) y[j] += xv * w[k * n_out + j];
    }
}
static void rms_w(float *out, const float *x, const float *w, int64_t n, float eps) { /* ops/norms.rs:13-29 */
    float ss = 0.0f;
    for (int64_t i = 0; i < n; i++) ss += x[i] * x[i];
    float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int64_t i = 0; i < n; i++) out[i] = x[i] * inv * w[i];
}

static const float *m3_layer_step(float *temporal, const float *p, float *ssm, float *kst, float *vst,
                                  float *angle, const m3cfg_t *c, float *taps) {
    const float EPS = 1e-5f;                                               /* ops/fast_math.rs:17 */
    int64_t dm = c->dm, ds = c->ds, hd = c->hd, ng = c->ng, di = dm * c->expand, nh = di / hd;
    int64_t ip = m3_ip(c), nr = c->n_rope;
    const float *norm_w = p; p += dm;
    const float *in_w = p; p += dm * ip;
    const float *dt_bias = p; p += nh;
    const float *bnw = p; p += ds;
    const float *cnw = p; p += ds;
    const float *b_bias = p; p += nh * ds;
    const float *c_bias = p; p += nh * ds;
    const float *Dp = p; p += nh;
    const float *ngw = p; p += di;
    const float *out_w = p; p += di * dm;
    float *normed = (float *)malloc(sizeof(float) * (dm + ip + 2 * ng * ds + 2 * di + dm));
    float *proj = normed + dm, *bn = proj + ip, *cn = bn + ng * ds, *yv = cn + ng * ds, *gated = yv + di, *out = gated + di;
    rms_w(normed, temporal, norm_w, dm, EPS);                              /* :93-98 */
    gemv_rm(proj, normed, in_w, dm, ip);                                   /* :101-108 */
    const float *z = proj, *x = proj + di, *braw = proj + 2 * di, *craw = braw + ng * ds; /* :111-127 */
    int64_t dd_dt = 2 * di + 2 * ng * ds, dd_a = dd_dt + nh, tr = dd_a + nh, ang = tr + nh;
    for (int64_t g = 0; g < ng; g++) {                                     /* bcnorm, ops/norms.rs:50-80 */
        rms_w(bn + g * ds, braw + g * ds, bnw, ds, EPS);
        rms_w(cn + g * ds, craw + g * ds, cnw, ds, EPS);
    }
    float tanh_pi[64];
    for (int64_t a = 0; a < nr; a++) tanh_pi[a] = tanhf(proj[ang + a]) * 3.14159265358979323846f; /* :156-162 */
    for (int64_t h = 0; h < nh; h++) {
        int64_t g = h / (nh / ng);
        float a_val = fminf(-heavy_tail(proj[dd_a + h]), -c->a_floor);     /* :168 */
        float dt_val = softplus_cpu(proj[dd_dt + h] + dt_bias[h]);         /* :171 */
        float kl[256], ql[256];
        for (int64_t n = 0; n < ds; n++) {                                 /* :174-179 */
            kl[n] = bn[g * ds + n] + b_bias[h * ds + n];
            ql[n] = cn[g * ds + n] + c_bias[h * ds + n];
        }
        for (int64_t a = 0; a < nr; a++) {                                 /* :182-206 */
            float delta = tanh_pi[a] * dt_val;
            double acc = (double)angle[h * nr + a] + (double)delta;
            const double two_pi = 2.0 * 3.14159265358979323846;
            acc -= two_pi * floor(acc / two_pi);
            angle[h * nr + a] = (float)acc;
            float sn = sinf(angle[h * nr + a]), cs = cosf(angle[h * nr + a]);
            float b0 = kl[2 * a], b1 = kl[2 * a + 1];
            kl[2 * a] = cs * b0 - sn * b1; kl[2 * a + 1] = sn * b0 + cs * b1;
            float c0 = ql[2 * a], c1 = ql[2 * a + 1];
            ql[2 * a] = cs * c0 - sn * c1; ql[2 * a + 1] = sn * c0 + cs * c1;
        }
        float alpha = orc_fast_exp(a_val * dt_val);                        /* :209-212 */
        float trap = 1.0f / (1.0f + orc_fast_exp(-proj[tr + h]));
        float beta = alpha * dt_val * (1.0f - trap);
        float gamma = trap * dt_val;
        if (taps) {
            taps[0 * nh + h] = alpha; taps[1 * nh + h] = beta; taps[2 * nh + h] = gamma;
            taps[3 * nh + h] = dt_val; taps[4 * nh + h] = trap; taps[5 * nh + h] = a_val;
            memcpy(taps + 6 * nh + h * ds, kl, sizeof(float) * ds);
            memcpy(taps + 6 * nh + nh * ds + h * ds, ql, sizeof(float) * ds);
        }
        const float *kp = kst + h * ds;
        for (int64_t pp = 0; pp < hd; pp++) {                              /* :215-231, forward.rs:85-138 */
            float xv = x[h * hd + pp], bv = beta * vst[h * hd + pp], gx = gamma * xv;
            float *H = ssm + (h * hd + pp) * ds;
            float yacc = 0.0f;
            for (int64_t n = 0; n < ds; n++) {
                H[n] = fmaf(alpha, H[n], fmaf(bv, kp[n], gx * kl[n]));
                yacc = fmaf(H[n], ql[n], yacc);
            }
            yv[h * hd + pp] = fmaf(Dp[h], xv, yacc);
        }
        memcpy(kst + h * ds, kl, sizeof(float) * ds);                      /* :234-237 */
        for (int64_t pp = 0; pp < hd; pp++) vst[h * hd + pp] = x[h * hd + pp];
    }
    if (c->outproj_norm) {                                                 /* rmsnorm_gated, ops/norms.rs:84-114 */
        for (int64_t g0 = 0; g0 < di; g0 += hd) {
            float ss = 0.0f;
            for (int64_t i = g0; i < g0 + hd; i++) ss += yv[i] * yv[i];
            float inv = 1.0f / sqrtf(ss / (float)hd + EPS);
            for (int64_t i = g0; i < g0 + hd; i++) {
                float zi = z[i];
                gated[i] = yv[i] * inv * ngw[i] * (zi / (1.0f + orc_fast_exp(-zi)));
            }
        }
    } else {
        for (int64_t i = 0; i < di; i++) {                                 /* :248-253 */
            float zi = z[i];
            float sig = 1.0f / (1.0f + orc_fast_exp(-zi));
            gated[i] = yv[i] * zi * sig;
        }
    }
    gemv_rm(out, gated, out_w, di, dm);                                    /* :256-267 */
    for (int64_t i = 0; i < dm; i++) temporal[i] = out[i] + temporal[i];
    free(normed);
    return p;
}

/* Backbone step (src/mamba3_siso/cpu/inference.rs:262-298): input_proj -> layers -> norm_f.
 * States are [L][...] blocks. taps (optional): [L][6*nh + 2*nh*ds]. */
ORC_API void orc_m3_backbone_step(float *temporal, const float *input, const float *params, float *ssm,
                                  float *kst, float *vst, float *angle, float *taps, int64_t dm,
                                  int64_t ds, int64_t expand, int64_t hd, int64_t ng, int64_t n_layers,
                                  int64_t n_rope, float a_floor, int outproj_norm, int64_t input_dim) {
    m3cfg_t c = { dm, ds, expand, hd, ng, n_layers, n_rope, a_floor, outproj_norm };
    int64_t di = dm * expand, nh = di / hd, na = n_rope > 0 ? n_rope : 1;
    const float *p = params;
    const float *ipw = p; p += input_dim * dm;
    const float *ipb = p; p += dm;
    gemv_rm(temporal, input, ipw, input_dim, dm);
    for (int64_t i = 0; i < dm; i++) temporal[i] += ipb[i];
    for (int64_t l = 0; l < n_layers; l++)
        p = m3_layer_step(temporal, p, ssm + l * nh * hd * ds, kst + l * nh * ds, vst + l * nh * hd,
                          angle + l * nh * na, &c, taps ? taps + l * (6 * nh + 2 * nh * ds) : NULL);
    float *tmp = (float *)malloc(sizeof(float) * dm);
    rms_w(tmp, temporal, p, dm, 1e-5f);
    memcpy(temporal, tmp, sizeof(float) * dm);
    free(tmp);
}
