// Shared device/host helpers for libmamba_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/mamba_hip.h"

namespace mrs {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// ---- storage types ---------------------------------------------------------
// Activations are stored as f32, IEEE f16 or bf16 and widened to f32 on load;
// stores round to nearest even (gfx950 has v_cvt_pk_bf16_f32 for bf16).
using f16_t = _Float16;
using bf16_t = __bf16;

template <typename T> struct Store;
template <> struct Store<float> {
    static constexpr int dtype = MRS_F32;
    __device__ static __forceinline__ float ld(const float *p) { return *p; }
    __device__ static __forceinline__ void st(float *p, float v) { *p = v; }
};
template <> struct Store<f16_t> {
    static constexpr int dtype = MRS_F16;
    __device__ static __forceinline__ float ld(const f16_t *p) { return (float)*p; }
    __device__ static __forceinline__ void st(f16_t *p, float v) { *p = (f16_t)v; }
};
template <> struct Store<bf16_t> {
    static constexpr int dtype = MRS_BF16;
    __device__ static __forceinline__ float ld(const bf16_t *p) {
        return __uint_as_float((uint32_t)(*reinterpret_cast<const uint16_t *>(p)) << 16);
    }
    __device__ static __forceinline__ void st(bf16_t *p, float v) { *p = (bf16_t)v; }
};

// 2^x on the transcendental unit (v_exp_f32).  Arguments here are <= 0 or small,
// results below the f32 normal range flush to 0, which is what the recurrence wants.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// x * sigmoid(x) = x / (1 + 2^(-x log2 e)); rcp is 1 ulp.  For x -> -inf the
// denominator overflows to +inf and the product is -0, the correct limit.
__device__ __forceinline__ float silu(float x) { return x * fast_rcp(1.0f + fast_exp2(-x * kLog2e)); }

// softplus with the reference's pass-through above 20 (kernels/activations.cu:39): log(1 + e^v) on the
// transcendental unit.  Below e = 0.03 the sum 1 + e would drop e's low bits, so log1p's series takes over
// (next term e^6/6 < 1.3e-10); above it the rounding of 1 + e is at most 2e-6 of the result.
__device__ __forceinline__ float softplus20(float v) {
    if (v > 20.0f) return v;
    const float e = fast_exp2(v * kLog2e);
    const float series = e * fmaf(e, fmaf(e, fmaf(e, fmaf(e, 0.2f, -0.25f), 0.33333334f), -0.5f), 1.0f);
    const float vialog = __builtin_amdgcn_logf(1.0f + e) * 0.6931471805599453f;
    return e < 0.03f ? series : vialog;
}

// Workgroup barrier that publishes LDS writes only: global loads issued before it stay in flight across it (the
// ordinary barrier's fence waits for every outstanding memory operation of the wave).  Not for data that travels
// through global memory.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// softplus for a result that is stored in 16 bits (8 or 11 significant bits), as max(v, 0) + log(1 + e^-|v|): no overflow,
// so no clamp, and above 20 the sum 1 + e^-|v| is 1 and the result is v itself, the reference's pass-through
// (kernels/activations.cu:39).  log(1 + t) on the transcendental unit is off by at most 2^-24 / t relative to itself,
// i.e. below 2^-12 of the result for t >= 2^-12; under that (v < -12 ln 2) the result is t to 2^-13.  Eight issue slots,
// two of them transcendental (the clamped form with log1p's second term and two selects took twelve).
__device__ __forceinline__ float softplus20_16(float v) {
    const float t = fast_exp2(-fabsf(v) * kLog2e);
    const float r = fmaf(__builtin_amdgcn_logf(1.0f + t), 0.6931471805599453f, fmaxf(v, 0.0f));
    return v < -8.317766f ? t : r;
}

// ---- host-side error plumbing ---------------------------------------------
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);

// Internal launchers shared with the backbone engine (strides and fusions the public entry points do not expose).
// StepFold: the step kernel forms the x_proj row itself from per-tile shares [n_tiles][rows][xd] f32 (summed in tile
// order, rounded to the storage type); dt input at element 0, B at b_off, C at c_off of the row.
// y_mt != 0: y is written in the tiled order of tiled_a_index (y_mt row tiles) instead of row-major.
struct StepFold { const float *xpart; int n_tiles, rows, xd, b_off, c_off, y_mt; };
// Element (row, k) of an activation matrix stored as the matrix-core A operand in lane order -- [k-step][row tile][lane][8],
// lane = row % 16 + 16 * ((k % 32) / 8), mt row tiles of 16 rows -- so that a wave's load of one operand piece is one
// contiguous kilobyte (gemm_wide.hip reads it; the kernels that produce such a matrix write it this way).
__host__ __device__ inline int64_t tiled_a_index(int row, int k, int mt) {
    return ((((int64_t)(k >> 5) * mt + (row >> 4)) * 64 + (row & 15) + 16 * ((k >> 3) & 3)) << 3) + (k & 7);
}
int launch_ssm_step_fused(hipStream_t st, int dtype, float *h, void *y, const void *delta, const float *dt_bias,
                          const void *dt_in, const void *dt_w, int dr, int dt_transposed, const void *u, const void *Bb, const void *Cb, int64_t bc_stride, const void *gate,
                          int64_t gate_stride, int gate_mode, const float *a_neg, const float *D, int batch,
                          int di, int ds, const StepFold *fold = nullptr, int y_mt = 0);
int launch_conv1d_step(hipStream_t st, int dtype, void *out, float *state, const void *new_x, int64_t x_stride,
                       const float *weight, const float *bias, int batch, int d_inner, int d_conv, int apply_silu);

// Skinny (M <= 128) 16-bit GEMM on a transposed weight, with the decode chain's fused prologue / epilogues.
struct SkinnyEpi {
    int mode;            // 0: store C
                         // 1: in_proj  -- conv step + SiLU on columns < di, gate columns stored
                         // 2: out_proj -- residual[row, col] += round(C); per-row sums of squares of the new
                         //                residual over this workgroup's 16 columns go to partials[row][column tile]
    float *conv_state;   // [M][di][dc]                                  (mode 1)
    const float *conv_w, *conv_b;
    void *u;             // [M][di], activation type
    int di, dc;
    float *residual;     // [M][N] f32, updated in place                 (mode 2)
    float *partials;     // [M][n_partials] f32: written by mode 2, read when row_scale is set
    int n_partials;
    const float *next_norm_w;  // mode 2: norm weight of the layer after, or null (last layer)
    void *prenorm;       // mode 2: [M][N] activation type, round(residual * next_norm_w): the next in_proj's operand
    // RMSNorm folded around the product: A = round(residual * norm_w) and the sums are scaled by
    // 1/rms[row], rms from the row's partials (row_scale != 0)
    int row_scale;
    float eps;
    // mode 1, optional: x_proj's products ride in the same launch (a few rows only).  Every x-half workgroup leaves its
    // 16 columns' share u[row, 16 cols] . xw[16 rows, xd] in xpart[tile][row][xd]; the step kernel sums the tiles.
    const void *xw;      // [di][xd] activation type (row-major, not transposed), or null
    int xd;
    float *xpart;        // [di / 16][M][xd] f32
    // mode 0, optional: K split over ksplit workgroups per tile (grid z), each leaving its f32 share in
    // xpart[slice][M][N] -- the layout above, so the same reader sums them (a long K with few output tiles:
    // x_proj of a wide model is 12 tiles over K = 5120)
    int ksplit;
    int kslice;          // set by the launcher: 32-wide k-steps per slice
    // tiled route (gemm_wide.hip) and matrix-core route of gemm_skinny.hip: A is stored [k-step][row tile][lane][8] -- the matrix-core operand in lane order, 16-row
    // tiles (tiled_a_index), rows past M present with any contents -- instead of row-major
    int a_tiled;
    int prenorm_mt;      // mode 2: != 0 writes prenorm in that tiled order (prenorm_mt row tiles) for the next tiled in_proj
    // matrix-core route of gemm_skinny.hip: the weight is the tiled copy (launch_tile_weight) instead of Wt[N][K]
    int w_tiled;
    // mode 1, optional: a second copy of u in tiled order (u_tiled_mt row tiles), the operand of a tiled x_proj
    void *u_tiled;
    int u_tiled_mt;
};
// The same products from a TILED weight (gemm_wide.hip): up to 64 rows over a weight of megabytes.  Wp holds the 16 columns x 32 k
// of each matrix-core operand as 1 KB in lane order, column tile by column tile (launch_tile_weight builds it from the
// transposed weight Wt[N][K]; tiled_weight_elems() elements, columns padded to a multiple of 16).  Same epilogues, except
// the x_proj shares (SkinnyEpi::xw, ksplit).
bool tiled_gemm_ok(int dtype, int M, int N, int K, int64_t lda, const void *A, const void *Wp);
size_t tiled_weight_elems(int N, int K);
int launch_tile_weight(hipStream_t st, int dtype, void *Wp, const void *Wt, int N, int K);
int launch_tiled_gemm(hipStream_t st, int dtype, void *C, int out_f32, int64_t ldc, const void *A, int64_t lda, const void *Wp, int M,
                      int N, int K, const SkinnyEpi &ep);
int skinny_max_rows();   // rows the 16-bit matrix-core route takes (128; MRS_SKINNY_MAX_ROWS overrides)
bool skinny_gemm_ok(int dtype, int M, int N, int K, int64_t lda, const void *A, const void *Wt);
int launch_skinny_gemm(hipStream_t st, int dtype, void *C, int out_f32, int64_t ldc, const void *A, int64_t lda, const void *Wt,
                       int M, int N, int K, const SkinnyEpi &ep);
int launch_transpose(hipStream_t st, int dtype, void *Wt, const void *W, int K, int N);
// delta[r, d] = softplus(round(dt_in[r, :] . wt[d, :]) + bias[d]) for 16-bit storage; wt is the transposed [d_inner][dt_rank] weight
// A whole f32 backbone step in one launch for small models (one workgroup per batch row; csrc/tiny_step.hip).  All
// pointers are device memory; weights row-major as the engine holds them (in_proj [dm][2 di], x_proj [di][xd],
// dt_w [dt_rank][di], out_proj [di][dm], in_w [input_dim][dm] or null for the identity input projection).
struct TinyStepLayer {
    const float *norm_w, *in_proj, *conv_w, *conv_b, *x_proj, *dt_w, *dt_b, *a_neg, *D, *out_proj;
};
struct TinyStepArgs {
    const TinyStepLayer *layers;
    const float *input, *in_w, *in_b, *norm_f;
    float *conv_state, *ssm_state, *temporal;
    float eps;
    int n_layers, batch, input_dim, dm, di, ds, dc, dr, xd;
};
// The same for the Mamba-3 SISO backbone (csrc/tiny_m3_step.hip): in_proj [dm][ip], out_proj [di][dm] row-major f32;
// states as the engine holds them ([layer][batch]...).
struct TinyM3StepLayer {
    const float *norm_w, *in_proj, *dt_bias, *bnw, *cnw, *b_bias, *c_bias, *D, *ngw, *out_proj;
};
struct TinyM3StepArgs {
    const TinyM3StepLayer *layers;
    const float *input, *in_w, *in_b, *norm_f;
    float *ssm, *kst, *vst, *angle, *temporal;
    float eps, a_floor;
    int n_layers, batch, input_dim, dm, di, nh, hd, ds, ng, nr, ip, outproj_norm;
};
bool tiny_m3_step_ok(int dtype, int input_dim, int dm, int di, int nh, int hd, int ds, int ng, int nr, int ip);
int launch_tiny_m3_step(hipStream_t st, const TinyM3StepArgs &a);
bool tiny_step_ok(int dtype, int input_dim, int dm, int di, int ds, int dc, int dr, int xd);
int launch_tiny_step(hipStream_t st, const TinyStepArgs &a);
bool dt_proj_softplus_ok(int dtype, int di, int dr, int64_t xs, const void *delta, const void *dt_in, const void *wt);
int launch_dt_proj_softplus(hipStream_t st, int dtype, void *delta, const void *dt_in, int64_t xs, const void *wt, const float *bias,
                            int64_t rows, int di, int dr);
// partials[row][0] = sum_k x[row][k]^2, partials[row][1..n_partials) = 0; prenorm[row][k] = round(x[row][k] * w[k])
// a_mt != 0: prenorm is written in the tiled order of tiled_a_index with a_mt row tiles
int launch_prenorm_rows(hipStream_t st, int dtype, float *partials, int n_partials, void *prenorm, const float *x, float *copy_to,
                        const float *w, int M, int K, int a_mt = 0);

// mrs_m3_ssd_fwd with x read in place out of wider rows (x_stride elements apart, 0 = dense; 16-bit storage only).
// With `gen` the kernel forms K and Q itself (K and Q are not read and may be null): K = rot(angle, bn + b_bias[head]),
// Q = rot(angle, cn + c_bias[head]) with bn / cn the normalised and weighted B / C rows (storage type, bc_stride elements
// apart -- the reference's bcnorm_fwd_* stores them in the activation type as well, kernels/mamba3_ops.cu:1193-1230),
// angle [batch, T, nheads, n_rope] and the first n_rope pairs of a row turned.  headdim = d_state = 64, 16-bit storage.
// head_major: the caller keeps what the kernel reads per (head, step) with the steps of a head next to each other --
// dt, trap, a_val as [batch, nheads, T] and angle as [batch, nheads, T, n_rope] -- so a chunk's 64 steps are a few whole
// cache lines instead of a piece of 64 different ones.
// gate: when not null, y leaves as y * silu(gate) (rows of gate_stride elements in the storage type, the first nheads *
// headdim of each used) -- the plain SiLU gate of the layer, folded into the store of the output tile.
struct SsdGenArgs { const void *bn, *cn; int64_t bc_stride; const float *angle, *b_bias, *c_bias; int n_rope; int head_major;
                    const void *gate; int64_t gate_stride; };
int m3_ssd_fwd_ex(void *stream, int dtype, float *ssm_state, float *k_state, float *v_state, void *y, const void *x,
                  int64_t x_stride, const void *K, const void *Q, const float *dt, const float *trap, const float *a_val,
                  const float *D, void *workspace, size_t workspace_bytes, unsigned flags, int batch, int T, int nheads,
                  int headdim, int d_state, int chunk_size, const SsdGenArgs *gen = nullptr);

// What the LM loop (embedding gather, head, argmax / sampling, generation bookkeeping) needs from a backbone engine;
// the Mamba-1 and the Mamba-3 engine each fill one in.  All functions are stream-ordered on `stream`.
struct LmHooks {
    void *self;
    int batch, d_model, dtype, identity_proj;
    hipStream_t stream;
    void *blas;               // rocblas_handle of the engine
    float *d_input;           // [batch, d_model] f32: the rows a step reads
    float *temporal;          // [batch, d_model] f32: final-norm output of the last step / prefill
    void *temporal_t;         // the same in the storage type, or null when the engine keeps no such copy
    int (*step)(void *self);                         // one decode step (capturable: launches only)
    int (*reset)(void *self);
    size_t (*state_bytes)(void *self);               // recurrent state, for save / restore around a warm-up run
    int (*state_copy)(void *self, void *buf, int restore);
    int (*prefill)(void *self, const int *dev_tokens, const void *embed, int vocab, int T);   // tokens [batch, T] on device
};
// gathers rows of the embedding table (storage type) as f32: out[r, :] = embed[clamp(tokens[r]), :] (engine prefill staging)
int launch_embed_gather(hipStream_t st, int dtype, float *out, const void *embed, const int *tokens, int64_t rows, int dm, int vocab);

// sample_token for every active row (sampling.hip); all pointers device memory
int launch_sample_rows(hipStream_t st, int *tokens, const float *logits, float *work, int64_t ld, int rows, int vocab,
                       const mrs_sampler *samplers, const unsigned *seen, unsigned long long *rng, const int *active);

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

}  // namespace mrs

// The LM loop over any engine that fills in the hooks (engine.hip); `fn` names the caller in error messages.
int mrs_lm_create_from_hooks(mrs_lm **out, const mrs::LmHooks &eng, const float *embed, int vocab, const char *fn);

// Dispatch a templated launch on the activation storage type.
#define MRS_DISPATCH_DTYPE(dtype, T, ...)                                         \
    switch (dtype) {                                                              \
        case MRS_F32: { using T = float; __VA_ARGS__; break; }                    \
        case MRS_F16: { using T = mrs::f16_t; __VA_ARGS__; break; }               \
        case MRS_BF16: { using T = mrs::bf16_t; __VA_ARGS__; break; }             \
        default: return mrs::fail(MRS_E_DTYPE, "dtype %d is not f32/f16/bf16", (int)(dtype)); \
    }
