// Mamba-1 backbone and LM engines: the host-side surface of the reference's
// GpuMambaBackbone (src/mamba_ssm/gpu/inference.rs:1515-1855) and the greedy loop of
// GpuMambaLM (src/module/gpu_lm.rs:323-377), driving the kernels of this library.
//
// Ownership follows the reference (inference.rs:92-143): the engine owns its weights
// (bulk projection matrices in the storage dtype, everything else f32), the persistent
// conv/SSM state and every scratch buffer; step() allocates nothing.  The residual
// stream, states, a_neg, D, biases and norm weights stay f32 (inference.rs:150-165).
//
// Decode, per layer (the reference launches 10 kernels + 4 GEMMs, inference.rs:993-1252):
//   16-bit storage, batch <= 64: four kernels on the library's own skinny GEMM (gemm_skinny.hip) -- in_proj with the
//     RMSNorm folded around it and the conv step + SiLU as epilogue, x_proj, one kernel for dt_proj + dt-bias + softplus
//     + state update + B/C gather + SiLU gate, out_proj with the residual add as epilogue;
//   otherwise: residual-add + RMSNorm, in_proj (vendor GEMM), conv step + SiLU reading the x half of in_proj's output
//     in place, x_proj, the fused step kernel, out_proj.
// Prefill: add + RMSNorm, in_proj, conv over T, x_proj, dt_proj + bias + softplus (one matrix-core kernel for 16-bit
// storage), the selective scan reading B/C and the raw gate in place, out_proj.
#include "common.hpp"
#include "glue.hpp"
#include "gemm_tune.hpp"
#include <rocblas/rocblas.h>
#include <stdlib.h>
#include <new>
#include <vector>
#include <algorithm>

namespace mrs {

#define MRS_HIP(expr)                                                                         \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess) return fail(MRS_E_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
    } while (0)
#define MRS_BLAS(expr)                                                                  \
    do {                                                                                \
        rocblas_status s_ = (expr);                                                     \
        if (s_ != rocblas_status_success) return fail(MRS_E_HIP, "%s: rocblas status %d", #expr, (int)s_); \
    } while (0)
#define MRS_TRY(expr)          \
    do {                       \
        int rc_ = (expr);      \
        if (rc_) return rc_;   \
    } while (0)

static size_t esize(int dtype) { return dtype == MRS_F32 ? 4 : 2; }
static rocblas_datatype blas_type(int dtype) {
    return dtype == MRS_F32 ? rocblas_datatype_f32_r : dtype == MRS_F16 ? rocblas_datatype_f16_r : rocblas_datatype_bf16_r;
}

// ---- glue kernels -------------------------------------------------------------------

// out[i] = round_T(sum over the K slices of a split x_proj of part[slice][i]), slices added in order (the library chain's
// x_proj at 65 to 128 rows: a K-split launch of the own GEMM and this sum take 10 us where the vendor kernel for 128 x 192 x
// 5120 takes 15.7)
template <typename T>
__global__ __launch_bounds__(256) void sum_shares_kernel(T *__restrict__ out, const float *__restrict__ part, int slices, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = 0.0f;
    for (int k = 0; k < slices; k++) s += part[(int64_t)k * n + i];
    Store<T>::st(out + i, s);
}

// delta = softplus(raw + bias[d]) in place (dt_proj bias + softplus_forward, kernels/activations.cu:32-52).
// VEC elements per thread as one 16-byte access (VEC = 16 / sizeof(T), d_inner % VEC == 0), or one by one.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void bias_softplus_kernel(T *__restrict__ x, const float *__restrict__ bias, int64_t n, int di) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (i >= n) return;
    const int d0 = (int)(i % di);
    struct alignas(VEC * sizeof(T)) V { T v[VEC]; };
    V t = *reinterpret_cast<const V *>(x + i);
    float bv[VEC];
    if (VEC % 4 == 0) {   // d0 is a multiple of VEC: the bias values are aligned 16-byte vectors too
#pragma unroll
        for (int j = 0; j < VEC; j += 4) {
            const float4 b4 = *reinterpret_cast<const float4 *>(bias + d0 + j);
            bv[j] = b4.x; bv[j + 1] = b4.y; bv[j + 2] = b4.z; bv[j + 3] = b4.w;
        }
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) bv[j] = bias[d0 + j];
    }
#pragma unroll
    for (int j = 0; j < VEC; j++) Store<T>::st(&t.v[j], softplus20(Store<T>::ld(&t.v[j]) + bv[j]));
    *reinterpret_cast<V *>(x + i) = t;
}

__global__ __launch_bounds__(256) void exp_negate_k(float *__restrict__ a_neg, const float *__restrict__ a_log, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) a_neg[i] = -expf(a_log[i]);
}

// residual[r, :] = embed[token[r], :] widened to f32 (host-side embed_lookup of the reference, gpu_lm.rs:352-373, moved on device)
// rows with finished[r] != 0 get a zero vector (generate_batch feeds finished slots zeros, gpu_lm.rs:436-441)
template <typename T>
__global__ __launch_bounds__(256) void embed_gather_kernel(float *__restrict__ out, const T *__restrict__ embed,
                                                           const int *__restrict__ tokens, int64_t rows, int dm, int vocab,
                                                           const int *__restrict__ finished = nullptr) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * dm) return;
    const int64_t r = i / dm;
    if (finished && finished[r]) { out[i] = 0.0f; return; }
    int tok = tokens[r];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    out[i] = Store<T>::ld(embed + (int64_t)tok * dm + (i - r * dm));
}

// Greedy pick: index of the maximum logit, the LAST one among equals (Iterator::max_by,
// src/module/sample.rs:250-257).  Stage 1: kArgParts blocks per row reduce a slice each; stage 2 combines.
constexpr int kArgParts = 32;
__device__ __forceinline__ void argmax_block_reduce(float &best, int &bi) {
    __shared__ float sv[256];
    __shared__ int si[256];
    sv[threadIdx.x] = best; si[threadIdx.x] = bi;
    __syncthreads();
    for (int s = 128; s >= 1; s >>= 1) {
        if ((int)threadIdx.x < s) {
            const float ov = sv[threadIdx.x + s];
            const int oi = si[threadIdx.x + s];
            if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi > si[threadIdx.x])) { sv[threadIdx.x] = ov; si[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    best = sv[0]; bi = si[0];
}
__global__ __launch_bounds__(256) void argmax_part_kernel(float *__restrict__ pv, int *__restrict__ pi,
                                                          const float *__restrict__ logits, int vocab, int64_t stride) {
    const int row = blockIdx.x / kArgParts, part = blockIdx.x % kArgParts;
    const int per = (vocab + kArgParts - 1) / kArgParts;
    const int lo = part * per, hi = min(vocab, lo + per);
    const float *r = logits + (int64_t)row * stride;
    float best = -INFINITY;
    int bi = lo < vocab ? lo : vocab - 1;
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
        const float v = r[i];
        if (v >= best) { best = v; bi = i; }   // ascending i per thread: >= keeps the last maximum
    }
    argmax_block_reduce(best, bi);
    if (threadIdx.x == 0) { pv[blockIdx.x] = best; pi[blockIdx.x] = bi; }
}
__global__ __launch_bounds__(64) void argmax_final_kernel(int *__restrict__ tokens, const float *__restrict__ pv,
                                                          const int *__restrict__ pi) {
    const int row = blockIdx.x;
    float best = -INFINITY;
    int bi = 0;
    if (threadIdx.x < kArgParts) { best = pv[row * kArgParts + threadIdx.x]; bi = pi[row * kArgParts + threadIdx.x]; }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ov = __shfl_xor(best, m, kWave);
        const int oi = __shfl_xor(bi, m, kWave);
        if (ov > best || (ov == best && oi > bi)) { best = ov; bi = oi; }
    }
    if (threadIdx.x == 0) tokens[row] = bi;
}

// ---- generate_batch bookkeeping on the device (src/module/gpu_lm.rs:404-513) ------------------------------
constexpr int kMaxEos = 16;
struct GenSlots {            // per-slot arrays, [batch] each unless noted
    int *prompt_off, *prompt_len, *prompt_pos, *finished, *active, *max_tokens, *n_eos, *eos /*[batch, kMaxEos]*/, *out_len, *sampled;
    unsigned *seen;          // [batch, vocab] occurrences in the slot's seen list
    int *n_running;          // [1] slots not finished after the latest step
};
struct GenDyn {              // buffers that grow between calls; read through device memory so a captured step stays valid
    const int *prompts;
    int *out;
    int out_stride;
};

// Seen list of generate_streaming starts as the prompt (gpu_lm.rs:364).
__global__ __launch_bounds__(256) void gen_seen_prompt_kernel(GenSlots g, const GenDyn *__restrict__ dyn, int batch, int vocab) {
    const int slot = blockIdx.y;
    const int n = g.prompt_len[slot];
    const int *p = dyn->prompts + g.prompt_off[slot];
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        const int t = p[i];
        if (t >= 0 && t < vocab) atomicAdd(&g.seen[(int64_t)slot * vocab + t], 1u);
    }
}

// After a step: slots still inside their prompt take the next prompt token; slots past it take the sampled token,
// unless it is an EOS id or max_tokens are out already -- then the slot is finished (gpu_lm.rs:494-511).  Also
// marks which slots sample after the next step (prompt consumed, not finished) and counts the running ones.
__global__ __launch_bounds__(1024) void gen_advance_kernel(GenSlots g, const GenDyn *__restrict__ dyn, int *__restrict__ last_token,
                                                           int batch, int vocab) {
    __shared__ int running;
    if (threadIdx.x == 0) running = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < batch; i += blockDim.x) {
        if (!g.finished[i]) {
            if (g.prompt_pos[i] < g.prompt_len[i]) {
                last_token[i] = dyn->prompts[g.prompt_off[i] + g.prompt_pos[i]];
                g.prompt_pos[i] += 1;
            } else {
                const int next = g.sampled[i];
                bool stop = g.out_len[i] >= g.max_tokens[i];
                for (int e = 0; e < g.n_eos[i]; e++) stop = stop || g.eos[i * kMaxEos + e] == next;
                if (stop) {
                    g.finished[i] = 1;
                } else {
                    dyn->out[(int64_t)i * dyn->out_stride + g.out_len[i]] = next;
                    g.out_len[i] += 1;
                    last_token[i] = next;
                    if (next >= 0 && next < vocab) g.seen[(int64_t)i * vocab + next] += 1u;
                }
            }
        }
        const int fin = g.finished[i];
        g.active[i] = !fin && g.prompt_pos[i] >= g.prompt_len[i];
        if (!fin) atomicAdd(&running, 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) *g.n_running = running;
}

}  // namespace mrs

using namespace mrs;

constexpr int64_t kFuseDtProjLimit = 4096;  // batch * dt_rank up to which dt_proj is folded into the decode step kernel

struct LayerDev {
    float *norm_w, *conv_w, *conv_b, *dt_b, *a_neg, *D;
    void *in_proj, *x_proj, *dt_w, *out_proj;
    void *dt_w_t;  // [d_inner][dt_rank] copy: the fused decode step (when dt_t_step) and the prefill dt_proj+softplus kernel read it
    int dt_t_step;
    void *in_proj_t, *x_proj_t, *out_proj_t;  // [N][K] copies: in / out for every 16-bit engine (own GEMM and vendor GEMM read them), x for the own chain only
    void *in_proj_p, *out_proj_p, *x_proj_p;  // tiled copies (launch_tile_weight): the own chain from two or three rows up
    int s4d;
};

constexpr int64_t kFoldXprojFloats = 1 << 20;   // largest [d_inner/16][rows][xdbl] block of shares the folded x_proj may use
constexpr int kMaxXprojSlices = 16;
// K slices of an x_proj launch of its own (0 = never split; MRS_DECODE_XPROJ_KSPLIT forces a count).  x_proj has few
// output tiles and a long K -- 12 workgroups over K = 5120 at 16 rows of the 2.8b shape -- so its K is cut into slices
// whose shares the step kernel sums, exactly as it sums the shares the in_proj launch leaves at few rows.
static int xproj_slices(int rows, int xd, int di) {
    static const int forced = getenv("MRS_DECODE_XPROJ_KSPLIT") ? atoi(getenv("MRS_DECODE_XPROJ_KSPLIT")) : -1;
    const int tiles = ((xd + 15) / 16) * ((rows + 15) / 16), nk = di / 32;
    int ks = forced >= 0 ? forced : 256 / tiles;
    ks = std::min(std::min(ks, kMaxXprojSlices), nk / 8);   // at least one k-step per wave
    return ks >= 2 ? ks : 1;
}

// Rows up to which x_proj rides in the in_proj launch (MRS_DECODE_FOLD_ROWS overrides).  Every step workgroup of a batch
// row re-reads that row's d_inner / 16 shares, so the sum grows with the batch while the launch it saves does not:
// measured at the 130m shape, the step went 420 -> 369 us at 8 rows, 467 -> 414 us at 16, even at 32, 622 -> 658 us at 64
// (1024-thread step workgroups, a quarter of the re-reads, were slower still: 701 us).
static int fold_rows_max() {
    static const int v = [] {
        if (getenv("MRS_DECODE_NO_FOLDED_XPROJ")) return 0;
        const char *e = getenv("MRS_DECODE_FOLD_ROWS");
        return e ? atoi(e) : 16;
    }();
    return v;
}
// ... and only while a row's shares stay small (30 KB at d_inner 1536): at d_inner 5120 they are 245 KB per row, re-read by
// each of the row's 80 step workgroups (2.8b-shape step at batch 1: 2.13 ms without the fold, 2.68 ms with it)
static bool narrow_model(int di, int xd) { return (int64_t)(di / 16) * xd * (int64_t)sizeof(float) <= 32768; }
static int fold_rows_for(int di, int xd) { return narrow_model(di, xd) ? fold_rows_max() : 0; }

struct Scratch {  // activations for M rows
    int64_t rows = 0;
    void *normed = nullptr, *proj = nullptr, *u = nullptr, *xdbl = nullptr, *delta = nullptr, *y = nullptr, *out = nullptr;
    float *residual = nullptr;
    float *partials = nullptr;  // [rows][d_model/16] row sums of squares, decode chain only
    void *u_tiled = nullptr;    // decode chain on tiled operands: u once more, in tile order (x_proj's operand)
    float *xpart = nullptr;     // decode chain: shares of the x_proj rows (per in_proj tile, or per K slice of x_proj)
    int64_t xpart_floats = 0;
    void *scan_ws = nullptr;
    size_t scan_ws_bytes = 0;
    int T = 0;
};

struct mrs_backbone {
    mrs_m1_config cfg;
    int input_dim, batch, dtype, di, dr, xd, identity_proj, device;
    const float *step_src;  // decode step: where layer 0 reads its input rows (null: the residual buffer itself)
    int split_xproj;  // library chain at up to 128 rows of a wide 16-bit model: x_proj as a K-split launch of the own GEMM
    int tiled;   // own chain from two (narrow models) or three rows up: the projections read tiled weights and tiled activation operands
    int wide;    // ... and in_proj / out_proj run on the column-tile kernel of gemm_wide.hip (wide models, up to 64 rows)
    int skinny;  // decode projections on the library's own GEMM (16-bit storage: batch <= 128 or 64, K % 32 == 0; f32: batch <= 4, K % 128 == 0)
    hipStream_t stream;
    rocblas_handle blas;
    GemmTuner *tuner;       // vendor-kernel choice for the prefill projections (off unless asked for)
    TinyStepLayer *tiny_layers;   // small f32 models: the layer table of the single-launch step (null: kernel chains)
    std::vector<LayerDev> layers;
    float *input_proj_w, *input_proj_b, *norm_f;
    std::vector<void *> allocs;
    std::vector<void *> prefill_allocs;  // the prefill scratch alone: released and re-made when the sequence length changes
    float *conv_state, *ssm_state;
    float *d_input, *temporal;
    void *temporal_t;  // decode: temporal once more in the storage type (16-bit engines), the LM head's operand
    Scratch step_s, prefill_s;
    float *prefill_in;  // [batch*T, input_dim] f32 staging for host input
    hipGraph_t graph;
    hipGraphExec_t graph_exec;
    int graph_ready;
};

static int dev_alloc(mrs_backbone *bb, void **p, size_t bytes) {
    MRS_HIP(hipMalloc(p, bytes ? bytes : 16));
    bb->allocs.push_back(*p);
    return MRS_OK;
}

static int upload_f32(mrs_backbone *bb, float **dst, const float *src, size_t n) {
    MRS_TRY(dev_alloc(bb, (void **)dst, n * sizeof(float)));
    MRS_HIP(hipMemcpyAsync(*dst, src, n * sizeof(float), hipMemcpyHostToDevice, bb->stream));
    return MRS_OK;
}

// Bulk matrix: upload f32, round to the storage dtype on device (RNE, as the reference's casts, kernels/elementwise.cu:17-38).
static int upload_bulk(mrs_backbone *bb, void **dst, const float *src, size_t n, float *stage) {
    MRS_HIP(hipMemcpyAsync(stage, src, n * sizeof(float), hipMemcpyHostToDevice, bb->stream));
    MRS_TRY(dev_alloc(bb, dst, n * esize(bb->dtype)));
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (bb->dtype == MRS_F32) MRS_HIP(hipMemcpyAsync(*dst, stage, n * 4, hipMemcpyDeviceToDevice, bb->stream));
    else if (bb->dtype == MRS_BF16) hipLaunchKernelGGL((cast_from_f32_kernel<bf16_t>), grid, block, 0, bb->stream, (bf16_t *)*dst, stage, (int64_t)n);
    else hipLaunchKernelGGL((cast_from_f32_kernel<f16_t>), grid, block, 0, bb->stream, (f16_t *)*dst, stage, (int64_t)n);
    MRS_HIP(hipStreamSynchronize(bb->stream));  // stage is reused by the next upload
    return check_launch("weight cast");
}

static int alloc_scratch(mrs_backbone *bb, Scratch *s, int64_t rows, int T) {
    const size_t es = esize(bb->dtype);
    const int dm = bb->cfg.d_model, di = bb->di, xd = bb->xd;
    s->rows = rows; s->T = T;
    MRS_TRY(dev_alloc(bb, (void **)&s->residual, rows * dm * sizeof(float)));
    // the tiled chain keeps the operands of in_proj and out_proj in 16-row tiles
    const int64_t rows16 = (T == 1 && bb->tiled) ? (rows + 15) / 16 * 16 : rows;
    MRS_TRY(dev_alloc(bb, &s->normed, rows16 * dm * es));
    MRS_TRY(dev_alloc(bb, &s->proj, rows * 2 * di * es));
    MRS_TRY(dev_alloc(bb, &s->u, rows * di * es));
    if (T == 1 && bb->tiled) MRS_TRY(dev_alloc(bb, &s->u_tiled, rows16 * di * es));
    MRS_TRY(dev_alloc(bb, &s->xdbl, rows * xd * es));
    MRS_TRY(dev_alloc(bb, &s->delta, rows * di * es));
    MRS_TRY(dev_alloc(bb, &s->y, rows16 * di * es));
    MRS_TRY(dev_alloc(bb, &s->out, rows * dm * es));
    if (T == 1) MRS_TRY(dev_alloc(bb, (void **)&s->partials, rows * (size_t)((dm + 15) / 16) * sizeof(float)));
    if (T == 1 && !bb->skinny && bb->split_xproj) {
        s->xpart_floats = (int64_t)kMaxXprojSlices * rows * xd;
        MRS_TRY(dev_alloc(bb, (void **)&s->xpart, (size_t)s->xpart_floats * sizeof(float)));
    }
    if (T == 1 && bb->skinny) {
        // shares of the x_proj rows: per 16-column tile of in_proj (few rows), else per K slice of a split x_proj
        int64_t need = (int64_t)kMaxXprojSlices * rows * xd;
        if (rows <= fold_rows_for(di, xd) && (int64_t)(di / 16) * rows * xd <= kFoldXprojFloats) need = std::max(need, (int64_t)(di / 16) * rows * xd);
        s->xpart_floats = need;
        MRS_TRY(dev_alloc(bb, (void **)&s->xpart, (size_t)need * sizeof(float)));
    }
    if (T > 1) {
        s->scan_ws_bytes = mrs_ssm_scan_workspace_bytes(bb->batch, T, di, bb->cfg.d_state);
        MRS_TRY(dev_alloc(bb, &s->scan_ws, s->scan_ws_bytes));
        // the flags of the one-launch scan start at zero here and every scan leaves them zero (MRS_SCAN_FLAGS_ZERO below)
        MRS_HIP(hipMemsetAsync(s->scan_ws, 0, std::min(s->scan_ws_bytes, mrs_ssm_scan_flag_bytes(bb->batch, di)), bb->stream));
    }
    return MRS_OK;
}

// C[M,N] = A[M,K] (row stride lda) . W[K,N], all row-major; f32 accumulate.
static int gemm_rm(mrs_backbone *bb, int dtype, void *C, int ldc, const void *A, int lda, const void *W, int M, int N, int K) {
    const rocblas_datatype t = blas_type(dtype);
    return gemm_ex_tuned(bb->tuner, bb->blas, bb->stream, 0, N, M, K, W, t, N, A, t, lda, C, t, ldc);
}

// The same product from the transposed copy Wt[N,K]: the vendor kernels for this operand order are faster at the prefill
// shapes (76 vs 84-92 us for in_proj at 16384 x 3072 x 768) and at decode row counts (128 x 2560 x 5120: 14.7 vs 46 us).
static int gemm_rm_t(mrs_backbone *bb, int dtype, void *C, int ldc, const void *A, int lda, const void *Wt, int M, int N, int K) {
    const rocblas_datatype t = blas_type(dtype);
    return gemm_ex_tuned(bb->tuner, bb->blas, bb->stream, 1, N, M, K, Wt, t, K, A, t, lda, C, t, ldc);
}

static int launch_add_rmsnorm(mrs_backbone *bb, float *residual, const void *add, void *out, bool out_f32, const float *w,
                              int64_t rows, int64_t out_stride, void *out2 = nullptr) {
    return launch_add_rmsnorm_any(bb->stream, bb->dtype, residual, add, out, out_f32, out2, w, bb->cfg.rms_norm_eps, rows, bb->cfg.d_model,
                                  out_stride);
}

// residual <- input (identity) or input . input_proj_w + b (f32 GEMM)
static int project_input(mrs_backbone *bb, float *residual, const float *input_dev, int64_t rows) {
    const int dm = bb->cfg.d_model;
    if (bb->identity_proj) {
        MRS_HIP(hipMemcpyAsync(residual, input_dev, rows * dm * sizeof(float), hipMemcpyDeviceToDevice, bb->stream));
        return MRS_OK;
    }
    // bias rows first, then accumulate the GEMM on top (beta = 1)
    {
        const int64_t n = rows * dm;
        hipLaunchKernelGGL(bias_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, bb->stream, residual, bb->input_proj_b, n, dm);
        MRS_TRY(check_launch("bias_rows_kernel"));
    }
    const float one = 1.0f;
    MRS_BLAS(rocblas_gemm_ex(bb->blas, rocblas_operation_none, rocblas_operation_none, dm, (int)rows, bb->input_dim, &one,
                             bb->input_proj_w, rocblas_datatype_f32_r, dm, input_dev, rocblas_datatype_f32_r, bb->input_dim,
                             &one, residual, rocblas_datatype_f32_r, dm, residual, rocblas_datatype_f32_r, dm,
                             rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0));
    return MRS_OK;
}

// The layer stack over `rows` = batch*T rows (T = 1: decode chain, T > 1: prefill chain), leaving the
// final-norm output of every row (decode) or of the last step of each sequence (prefill) in temporal [batch, dm] f32.
// Decode chain on the library's own GEMM for rows [r0, r0 + nr) of the batch, every layer, on stream st.  Three or
// four kernels per layer:
//   in_proj  on round(residual * norm_w) with the 1/rms row scale and the conv step + SiLU in its epilogue (only u and
//            the gate half are written); up to 16 rows its x-half workgroups also leave their shares of the x_proj rows,
//   x_proj   (above that row count),
//   dt_proj + softplus + scan step + gate (summing the x_proj shares first where they were left),
//   out_proj with the residual add as its epilogue, which also leaves each row's sum of squares (per 16-column tile)
//            and round(residual * next norm_w) for the next layer's in_proj.
// Rows are independent of each other from the first kernel to the last.  (Running the batch as two or four such chains
// of 16-32 rows on forked streams inside the graph was measured: the branches did not overlap -- 631 us for one chain of 64
// rows at the 130m shape, 722 us as two chains, 1112 us as four.)
static int decode_chain(mrs_backbone *bb, Scratch *s, int r0, int nr, hipStream_t st) {
    const int dm = bb->cfg.d_model, di = bb->di, ds = bb->cfg.d_state, dc = bb->cfg.d_conv, dr = bb->dr, xd = bb->xd;
    const int B = bb->batch, dt = bb->dtype, L = bb->cfg.n_layers, P = dm / 16;
    const size_t es = esize(dt);
    float *residual = s->residual + (size_t)r0 * dm, *partials = s->partials + (size_t)r0 * P;
    char *normed = (char *)s->normed + (size_t)r0 * dm * es, *proj = (char *)s->proj + (size_t)r0 * 2 * di * es;
    char *u = (char *)s->u + (size_t)r0 * di * es, *xdbl = (char *)s->xdbl + (size_t)r0 * xd * es;
    char *delta = (char *)s->delta + (size_t)r0 * di * es, *y = (char *)s->y + (size_t)r0 * di * es;
    char *out = (char *)s->out + (size_t)r0 * dm * es;
    float *xpart = s->xpart ? s->xpart + (size_t)r0 * (di / 16) * xd : nullptr;   // [tile][nr][xd] blocks, one per slice
    const char *z = proj + (size_t)di * es;  // gate half of in_proj's output
    // tiled chain (the whole batch as one chain): normed and y are stored as matrix-core operands in 16-row tiles
    const int a_mt = (bb->tiled && r0 == 0 && nr == B) ? (nr + 15) / 16 : 0;
    // batch * dt_rank up to which dt_proj rides in the step kernel.  On the tiled chain the alternative is an x_proj launch
    // that cannot split K (nobody would sum the shares): 12.5 us at 32 and 64 rows of the 2.8b shape, against 4.7 us split.
    // Per step at that shape, dt_proj in the step kernel / on its own: 32 rows 3.57 / 3.84 ms, 48 rows 4.32 / 4.34, 64 rows 5.04 / 4.89.
    static const int64_t wide_fuse = [] { const char *e = getenv("MRS_DECODE_FUSE_DT_LIMIT"); return e ? (int64_t)atoll(e) : (int64_t)6400; }();
    const int64_t fuse_limit = (a_mt && bb->wide) ? wide_fuse : kFuseDtProjLimit;
    for (int l = 0; l < L; l++) {
        const LayerDev &lw = bb->layers[l];
        float *conv = bb->conv_state + ((size_t)l * B + r0) * di * dc;
        float *ssm = bb->ssm_state + ((size_t)l * B + r0) * di * ds;
        if (l == 0) {
            const float *src = bb->step_src ? bb->step_src + (size_t)r0 * dm : residual;
            MRS_TRY(launch_prenorm_rows(st, dt, partials, P, normed, src, bb->step_src ? residual : nullptr, lw.norm_w, nr, dm, a_mt));
        }
        SkinnyEpi inp = {};
        inp.mode = 1; inp.conv_state = conv; inp.conv_w = lw.conv_w; inp.conv_b = lw.conv_b; inp.u = u; inp.di = di; inp.dc = dc;
        inp.row_scale = 1; inp.partials = partials; inp.n_partials = P; inp.eps = bb->cfg.rms_norm_eps;
        const bool fold_x = xpart && nr <= fold_rows_for(di, xd) && xd <= 256 && (int64_t)(di / 16) * nr * xd <= s->xpart_floats && lw.dt_t_step &&
                            di % (1024 / ds) == 0 && dr % 4 == 0 && (int64_t)nr * dr <= fuse_limit;
        if (fold_x) { inp.xw = lw.x_proj; inp.xd = xd; inp.xpart = xpart; }
        // x_proj as a launch of its own: K split into slices when the step kernel can sum the shares
        const bool step_sums = xpart && xd <= 256 && lw.dt_t_step && di % (1024 / ds) == 0 && dr % 4 == 0 && (int64_t)nr * dr <= fuse_limit;
        const int ksplit = (!fold_x && step_sums && dt != MRS_F32) ? xproj_slices(nr, xd, di) : 1;
        const StepFold fold = {xpart, fold_x ? di / 16 : ksplit, nr, xd, dr, dr + ds};
        if (a_mt) {
            inp.a_tiled = 1; inp.w_tiled = 1;
            if (!fold_x) { inp.u_tiled = s->u_tiled; inp.u_tiled_mt = a_mt; }
            if (bb->wide) MRS_TRY(launch_tiled_gemm(st, dt, proj, 0, 2 * di, normed, dm, lw.in_proj_p, nr, 2 * di, dm, inp));
            else MRS_TRY(launch_skinny_gemm(st, dt, proj, 0, 2 * di, normed, dm, lw.in_proj_p, nr, 2 * di, dm, inp));
        } else {
            MRS_TRY(launch_skinny_gemm(st, dt, proj, 0, 2 * di, normed, dm, lw.in_proj_t, nr, 2 * di, dm, inp));
        }
        const SkinnyEpi none = {};
        if (!fold_x) {
            SkinnyEpi xp = {};
            if (ksplit > 1) { xp.ksplit = ksplit; xp.xpart = xpart; }
            if (a_mt) {
                xp.a_tiled = 1; xp.w_tiled = 1;
                MRS_TRY(launch_skinny_gemm(st, dt, xdbl, 0, xd, s->u_tiled, di, lw.x_proj_p, nr, xd, di, xp));
            } else {
                MRS_TRY(launch_skinny_gemm(st, dt, xdbl, 0, xd, u, di, lw.x_proj_t, nr, xd, di, xp));
            }
        }
        if ((int64_t)nr * dr > fuse_limit && lw.dt_w_t && skinny_gemm_ok(dt, nr, di, dr, xd, xdbl, lw.dt_w_t)) {
            // wide dt_rank at a large batch: dt_proj as a GEMM of its own, bias + softplus in the step kernel
            MRS_TRY(launch_skinny_gemm(st, dt, delta, 0, di, xdbl, xd, lw.dt_w_t, nr, di, dr, none));
            MRS_TRY(launch_ssm_step_fused(st, dt, ssm, y, delta, lw.dt_b, nullptr, nullptr, 0, 0, u, xdbl + es * dr, xdbl + es * (dr + ds), xd, z,
                                          2 * di, 2, lw.a_neg, lw.D, nr, di, ds, nullptr, a_mt));
        } else {
            MRS_TRY(launch_ssm_step_fused(st, dt, ssm, y, delta, lw.dt_b, xdbl, lw.dt_t_step ? lw.dt_w_t : lw.dt_w, dr, lw.dt_t_step, u,
                                          xdbl + es * dr, xdbl + es * (dr + ds), xd, z, 2 * di, 2, lw.a_neg, lw.D, nr, di, ds,
                                          (fold_x || ksplit > 1) ? &fold : nullptr, a_mt));
        }
        SkinnyEpi outp = {};
        outp.mode = 2; outp.residual = residual; outp.partials = partials; outp.n_partials = P;
        outp.next_norm_w = l + 1 < L ? bb->layers[l + 1].norm_w : nullptr; outp.prenorm = normed;
        if (a_mt) {
            outp.a_tiled = 1; outp.w_tiled = 1; outp.prenorm_mt = a_mt;
            if (bb->wide) MRS_TRY(launch_tiled_gemm(st, dt, out, 0, dm, y, di, lw.out_proj_p, nr, dm, di, outp));
            else MRS_TRY(launch_skinny_gemm(st, dt, out, 0, dm, y, di, lw.out_proj_p, nr, dm, di, outp));
        } else {
            MRS_TRY(launch_skinny_gemm(st, dt, out, 0, dm, y, di, lw.out_proj_t, nr, dm, di, outp));
        }
    }
    return MRS_OK;
}

static int run_layers(mrs_backbone *bb, Scratch *s, int T) {
    const int dm = bb->cfg.d_model, di = bb->di, ds = bb->cfg.d_state, dc = bb->cfg.d_conv, dr = bb->dr, xd = bb->xd;
    const int B = bb->batch, dt = bb->dtype;
    const int64_t rows = (int64_t)B * T;
    const size_t es = esize(dt);
    const int L = bb->cfg.n_layers;
    if (T == 1 && bb->skinny) MRS_TRY(decode_chain(bb, s, 0, B, bb->stream));
    for (int l = 0; l < L && !(T == 1 && bb->skinny); l++) {
        const LayerDev &lw = bb->layers[l];
        float *conv = bb->conv_state + (size_t)l * B * di * dc;
        float *ssm = bb->ssm_state + (size_t)l * B * di * ds;
        const char *z = (const char *)s->proj + (size_t)di * es;  // gate half of in_proj's output
        const char *xb = (const char *)s->xdbl;
        MRS_TRY(launch_add_rmsnorm(bb, s->residual, l == 0 ? nullptr : s->out, s->normed, false, lw.norm_w, rows, dm));
        if (lw.in_proj_t) MRS_TRY(gemm_rm_t(bb, dt, s->proj, 2 * di, s->normed, dm, lw.in_proj_t, (int)rows, 2 * di, dm));
        else MRS_TRY(gemm_rm(bb, dt, s->proj, 2 * di, s->normed, dm, lw.in_proj, (int)rows, 2 * di, dm));
        if (T == 1) {
            MRS_TRY(launch_conv1d_step(bb->stream, dt, s->u, conv, s->proj, 2 * di, lw.conv_w, lw.conv_b, B, di, dc, 1));
            if (bb->split_xproj && lw.x_proj_p && s->xpart) {
                // few output tiles over a long K: the own GEMM with K cut into slices, then the slices added up
                const int tiles = ((xd + 15) / 16) * (((int)rows + 15) / 16);
                const int ksplit = std::max(2, std::min(std::min(kMaxXprojSlices, 768 / tiles), di / 32 / 8));
                SkinnyEpi xp = {};
                xp.ksplit = ksplit; xp.xpart = s->xpart; xp.w_tiled = 1;
                MRS_TRY(launch_skinny_gemm(bb->stream, dt, s->xdbl, 0, xd, s->u, di, lw.x_proj_p, (int)rows, xd, di, xp));
                const int64_t n = rows * xd;
                MRS_DISPATCH_DTYPE(dt, T_, hipLaunchKernelGGL((sum_shares_kernel<T_>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, bb->stream,
                                                              (T_ *)s->xdbl, s->xpart, ksplit, n));
                MRS_TRY(check_launch("sum_shares_kernel"));
            } else {
                MRS_TRY(gemm_rm(bb, dt, s->xdbl, xd, s->u, di, lw.x_proj, (int)rows, xd, di));
            }
            if ((int64_t)B * dr <= kFuseDtProjLimit) {
                // dt_proj (K = dt_rank) + bias + softplus + state update + B/C gather + SiLU gate: one kernel
                MRS_TRY(launch_ssm_step_fused(bb->stream, dt, ssm, s->y, s->delta, lw.dt_b, s->xdbl, lw.dt_t_step ? lw.dt_w_t : lw.dt_w, dr,
                                              lw.dt_t_step, s->u, xb + es * dr,
                                              xb + es * (dr + ds), xd, z, 2 * di, 2, lw.a_neg, lw.D, B, di, ds));
            } else {
                // large batch x dt_rank: every batch row would re-read the whole dt_proj weight inside the step kernel
                // (83 us at batch 128, d_inner 5120, dt_rank 160), so the projection goes to the library GEMM
                MRS_TRY(gemm_rm(bb, dt, s->delta, di, s->xdbl, xd, lw.dt_w, (int)rows, di, dr));
                MRS_TRY(launch_ssm_step_fused(bb->stream, dt, ssm, s->y, s->delta, lw.dt_b, nullptr, nullptr, 0, 0, s->u, xb + es * dr,
                                              xb + es * (dr + ds), xd, z, 2 * di, 2, lw.a_neg, lw.D, B, di, ds));
            }
        } else {
            MRS_TRY(mrs_conv1d_seq_silu(bb->stream, dt, s->u, conv, s->proj, 2 * di, lw.conv_w, lw.conv_b, B, T, di, dc));
            MRS_TRY(gemm_rm(bb, dt, s->xdbl, xd, s->u, di, lw.x_proj, (int)rows, xd, di));
            if (lw.dt_w_t && dt_proj_softplus_ok(dt, di, dr, xd, s->delta, s->xdbl, lw.dt_w_t)) {
                // dt_proj + bias + softplus in one matrix-core kernel (K = dt_rank is tiny: the op is one write of delta)
                MRS_TRY(launch_dt_proj_softplus(bb->stream, dt, s->delta, s->xdbl, xd, lw.dt_w_t, lw.dt_b, rows, di, dr));
            } else {
            MRS_TRY(gemm_rm(bb, dt, s->delta, di, s->xdbl, xd, lw.dt_w, (int)rows, di, dr));
            const int64_t n = rows * di;
            MRS_DISPATCH_DTYPE(dt, T_, {
                constexpr int VEC = 16 / (int)sizeof(T_);
                if (di % VEC == 0)
                    hipLaunchKernelGGL((bias_softplus_kernel<T_, VEC>), dim3((unsigned)((n / VEC + 255) / 256)), dim3(256), 0, bb->stream, (T_ *)s->delta, lw.dt_b, n, di);
                else
                    hipLaunchKernelGGL((bias_softplus_kernel<T_, 1>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, bb->stream, (T_ *)s->delta, lw.dt_b, n, di);
            });
            MRS_TRY(check_launch("bias_softplus_kernel"));
            }
            // ScanMode::use_parallel picks the route (src/mamba_ssm/gpu/prefill.rs:910-956)
            unsigned flags = MRS_GATE_SILU | MRS_SCAN_FLAGS_ZERO | (lw.s4d ? MRS_A_S4D_REAL : 0);
            // An explicit mode is honoured; in Auto the op picks the kernel itself (same recurrence, same tolerance).
            if (bb->cfg.scan_mode == MRS_SCAN_SEQUENTIAL) flags |= MRS_FORCE_SEQUENTIAL;
            else if (bb->cfg.scan_mode == MRS_SCAN_PARALLEL && ds == 16 && T >= 64) flags |= MRS_FORCE_PARALLEL;
            MRS_TRY(mrs_ssm_scan_fwd_ex(bb->stream, dt, ssm, s->y, s->delta, s->u, xb + es * dr, xb + es * (dr + ds), xd, lw.a_neg,
                                        lw.D, z, 2 * di, flags, s->scan_ws, s->scan_ws_bytes, B, T, di, ds));
        }
        if (lw.out_proj_t) MRS_TRY(gemm_rm_t(bb, dt, s->out, dm, s->y, di, lw.out_proj_t, (int)rows, dm, di));
        else MRS_TRY(gemm_rm(bb, dt, s->out, dm, s->y, di, lw.out_proj, (int)rows, dm, di));
    }
    if (T == 1) {
        // (the out_proj epilogue of the own-GEMM chain has already added the last layer's output)
        MRS_TRY(launch_add_rmsnorm(bb, s->residual, bb->skinny ? nullptr : s->out, bb->temporal, true, bb->norm_f, rows, dm,
                                   bb->dtype != MRS_F32 ? bb->temporal_t : nullptr));
    } else {
        // Only the last step of each sequence is kept (gather_last_timestep,
        // src/mamba_ssm/gpu/prefill.rs:1030-1046), so the final residual add + norm_f runs on those rows only.
        for (int b = 0; b < B; b++) {
            const size_t r = (size_t)b * T + (T - 1);
            MRS_TRY(launch_add_rmsnorm(bb, s->residual + r * dm, (const char *)s->out + r * dm * es, bb->temporal + (size_t)b * dm, true,
                                       bb->norm_f, 1, dm, bb->dtype != MRS_F32 ? (char *)bb->temporal_t + (size_t)b * dm * es : nullptr));
        }
    }
    return MRS_OK;
}

extern "C" int mrs_backbone_create(mrs_backbone **out, int gpu_ordinal, const mrs_m1_weights *w,
                                   const mrs_m1_config *cfg, int input_dim, int batch, int dtype) {
    if (!out || !w || !cfg || !w->layers || !w->norm_f_weight) return fail(MRS_E_NULL, "mrs_backbone_create: null pointer");
    if (dtype != MRS_F32 && dtype != MRS_F16 && dtype != MRS_BF16) return fail(MRS_E_DTYPE, "mrs_backbone_create: dtype %d", dtype);
    // MambaConfig::validate (src/config.rs:108-170)
    if (cfg->d_model < 1 || cfg->d_state < 1 || cfg->d_conv < 1 || cfg->expand < 1 || cfg->n_layers < 1)
        return fail(MRS_E_SHAPE, "mrs_backbone_create: d_model, d_state, d_conv, expand, n_layers must be > 0");
    const int64_t di64 = (int64_t)cfg->expand * cfg->d_model;
    if (cfg->d_model > (1 << 20) || cfg->n_layers > 4096 || di64 > 65535 || cfg->d_state > 256 || cfg->d_conv > 8 || di64 % 4 != 0)
        return fail(MRS_E_SHAPE, "mrs_backbone_create: config outside the reference's bounds (d_inner<=65535 and %%4==0, d_state<=256, d_conv<=8)");
    if (batch < 1 || input_dim < 1) return fail(MRS_E_SHAPE, "mrs_backbone_create: batch=%d input_dim=%d", batch, input_dim);
    const int identity = (w->input_proj_w == nullptr);
    if (identity && input_dim != cfg->d_model) return fail(MRS_E_SHAPE, "mrs_backbone_create: identity input_proj needs input_dim == d_model");
    mrs_backbone *bb = new (std::nothrow) mrs_backbone();
    if (!bb) return fail(MRS_E_HIP, "mrs_backbone_create: out of host memory");
    bb->cfg = *cfg; bb->input_dim = input_dim; bb->batch = batch; bb->dtype = dtype; bb->device = gpu_ordinal;
    bb->di = (int)di64; bb->dr = (cfg->d_model + 15) / 16; bb->xd = bb->dr + 2 * cfg->d_state; bb->identity_proj = identity;
    bb->graph_ready = 0; bb->graph = nullptr; bb->graph_exec = nullptr; bb->prefill_in = nullptr;
    bb->input_proj_w = nullptr; bb->input_proj_b = nullptr;
    *out = nullptr;
#define MRS_CREATE_TRY(expr) do { int rc_ = (expr); if (rc_) { mrs_backbone_destroy(bb); return rc_; } } while (0)
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
    const int dm = cfg->d_model, di = bb->di, ds = cfg->d_state, dc = cfg->d_conv, dr = bb->dr, xd = bb->xd, L = cfg->n_layers;
    size_t max_bulk = (size_t)dm * 2 * di;
    if ((size_t)di * xd > max_bulk) max_bulk = (size_t)di * xd;
    if ((size_t)di * ds > max_bulk) max_bulk = (size_t)di * ds;
    float *stage = nullptr;
    MRS_CREATE_TRY(dev_alloc(bb, (void **)&stage, max_bulk * sizeof(float)));
    if (!identity) {
        MRS_CREATE_TRY(upload_f32(bb, &bb->input_proj_w, w->input_proj_w, (size_t)input_dim * dm));
        if (w->input_proj_b) MRS_CREATE_TRY(upload_f32(bb, &bb->input_proj_b, w->input_proj_b, dm));
        else { MRS_CREATE_TRY(dev_alloc(bb, (void **)&bb->input_proj_b, dm * 4)); hipMemsetAsync(bb->input_proj_b, 0, dm * 4, bb->stream); }
    }
    bb->layers.resize(L);
    {
        static const bool off = [] { const char *e = getenv("MRS_DECODE_LIBRARY_GEMM"); return e && atoi(e) != 0; }();
        // Rows up to which the own chain beats the library chain (in_proj / out_proj from the transposed copies, default
        // vendor kernels), measured: 128 at the 130m shape (1032 vs 1091 us per step; at 256 rows 1490 vs 1392), 40 at the
        // 2.8b shape (32 rows 5.13 vs 8.35 ms, 40 rows 5.74 vs 5.92, 48 rows 6.13 vs 5.98, 64 rows 7.58 vs 6.19).  "Narrow"
        // as for the x_proj shares.
        // From two (narrow models) or three rows up the projections of the own chain run on the matrix cores and read TILED operands -- weights tiled at load,
        // activation operands written tiled by their producers.  On wide models in_proj / out_proj also run on the
        // column-tile kernel of gemm_wide.hip, which carries the own chain up to 64 rows there.
        static const bool no_tiled = [] { const char *e = getenv("MRS_DECODE_NO_TILED"); return e && atoi(e) != 0; }();
        static const int tiled_max_rows = [] { const char *e = getenv("MRS_DECODE_TILED_MAX_ROWS"); return e ? atoi(e) : 64; }();
        const bool pow2_state = ds == 4 || ds == 8 || ds == 16 || ds == 32 || ds == 64 || ds == 128 || ds == 256;
        // Below that the lanes-along-the-row route of the 16 x 16-tile GEMM is the faster one.  Per step, row-wise / tiled
        // matrix-core route: 130m shape 330 / 356 us at 1 row, 378 / 359 at 2, 420 / 370 at 4; 2.8b shape 1.90 / 2.22 ms at
        // 1 row, 2.08 / 2.25 at 2, 2.42 / 2.27 at 3, 2.48 / 2.31 at 4.
        static const int forced_min_rows = [] { const char *e = getenv("MRS_DECODE_TILED_MIN_ROWS"); return e ? atoi(e) : 0; }();
        const int tiled_min_rows = forced_min_rows > 0 ? forced_min_rows : (narrow_model(di, xd) ? 2 : 3);
        const bool can_tile = !off && !no_tiled && (dtype == MRS_BF16 || dtype == MRS_F16) && batch >= tiled_min_rows && dm % 32 == 0 && di % 32 == 0 && pow2_state;
        bb->wide = can_tile && batch <= std::min(tiled_max_rows, 64) && (int64_t)dm * 2 * di >= (int64_t)8 << 20 && !narrow_model(di, xd);
        const int max_rows = std::min(skinny_max_rows(), narrow_model(di, xd) ? 128 : (bb->wide ? 64 : 40));
        bb->skinny = !off && (dtype == MRS_BF16 || dtype == MRS_F16) && batch <= max_rows && dm % 32 == 0 && di % 32 == 0;
        bb->tiled = can_tile && bb->skinny;
        if (!bb->skinny) bb->wide = 0;
        bb->split_xproj = !off && !bb->skinny && (dtype == MRS_BF16 || dtype == MRS_F16) && batch <= 128 && di % 256 == 0 && xd % 8 == 0 &&
                          !narrow_model(di, xd);
        // f32 storage: the same chain on the row-wise route of the GEMM (one to four rows, rows of the operand in LDS)
        if (!off && dtype == MRS_F32 && batch <= 4 && dm % 128 == 0 && di % 128 == 0 && (int64_t)di * 16 <= 48 * 1024 &&
            getenv("MRS_DECODE_NO_ROWWISE") == nullptr)
            bb->skinny = 1;
    }
    int *flag = nullptr;
    MRS_CREATE_TRY(dev_alloc(bb, (void **)&flag, sizeof(int)));
    for (int l = 0; l < L; l++) {
        const mrs_m1_layer_weights &src = w->layers[l];
        LayerDev &d = bb->layers[l];
        if (!src.norm_weight || !src.in_proj_w || !src.conv1d_weight || !src.conv1d_bias || !src.x_proj_w || !src.dt_proj_w ||
            !src.dt_proj_b || !src.a_log || !src.d_param || !src.out_proj_w) {
            mrs_backbone_destroy(bb);
            return fail(MRS_E_NULL, "mrs_backbone_create: layer %d has a null weight", l);
        }
        MRS_CREATE_TRY(upload_f32(bb, &d.norm_w, src.norm_weight, dm));
        MRS_CREATE_TRY(upload_bulk(bb, &d.in_proj, src.in_proj_w, (size_t)dm * 2 * di, stage));
        MRS_CREATE_TRY(upload_f32(bb, &d.conv_w, src.conv1d_weight, (size_t)di * dc));
        MRS_CREATE_TRY(upload_f32(bb, &d.conv_b, src.conv1d_bias, di));
        MRS_CREATE_TRY(upload_bulk(bb, &d.x_proj, src.x_proj_w, (size_t)di * xd, stage));
        MRS_CREATE_TRY(upload_bulk(bb, &d.dt_w, src.dt_proj_w, (size_t)dr * di, stage));
        MRS_CREATE_TRY(upload_f32(bb, &d.dt_b, src.dt_proj_b, di));
        MRS_CREATE_TRY(upload_f32(bb, &d.D, src.d_param, di));
        MRS_CREATE_TRY(upload_bulk(bb, &d.out_proj, src.out_proj_w, (size_t)di * dm, stage));
        d.in_proj_t = d.x_proj_t = d.out_proj_t = d.dt_w_t = d.in_proj_p = d.out_proj_p = d.x_proj_p = nullptr;
        d.dt_t_step = (ds == 4 || ds == 8 || ds == 16 || ds == 32 || ds == 64 || ds == 128 || ds == 256) && dr % ds == 0 && xd % 4 == 0;
        if (d.dt_t_step || (bb->dtype != MRS_F32 && dr % 8 == 0)) {
            MRS_CREATE_TRY(dev_alloc(bb, &d.dt_w_t, (size_t)dr * di * esize(bb->dtype)));
            MRS_CREATE_TRY(launch_transpose(bb->stream, bb->dtype, d.dt_w_t, d.dt_w, dr, di));
        }
        if (bb->skinny || bb->dtype != MRS_F32) {
            // transposed copies (one more copy of the bulk weights in HBM): the decode chain's own GEMM reads them, and the
            // vendor kernels for this operand order are the faster ones for in_proj and out_proj from 128 rows up
            const size_t es_ = esize(bb->dtype);
            MRS_CREATE_TRY(dev_alloc(bb, &d.in_proj_t, (size_t)dm * 2 * di * es_));
            MRS_CREATE_TRY(dev_alloc(bb, &d.out_proj_t, (size_t)di * dm * es_));
            MRS_CREATE_TRY(launch_transpose(bb->stream, bb->dtype, d.in_proj_t, d.in_proj, dm, 2 * di));
            MRS_CREATE_TRY(launch_transpose(bb->stream, bb->dtype, d.out_proj_t, d.out_proj, di, dm));
        }
        if (bb->tiled) {
            const size_t es_ = esize(bb->dtype);
            MRS_CREATE_TRY(dev_alloc(bb, &d.in_proj_p, tiled_weight_elems(2 * di, dm) * es_));
            MRS_CREATE_TRY(dev_alloc(bb, &d.out_proj_p, tiled_weight_elems(dm, di) * es_));
            MRS_CREATE_TRY(launch_tile_weight(bb->stream, bb->dtype, d.in_proj_p, d.in_proj_t, 2 * di, dm));
            MRS_CREATE_TRY(launch_tile_weight(bb->stream, bb->dtype, d.out_proj_p, d.out_proj_t, dm, di));
        }
        if (bb->skinny || bb->split_xproj) {
            MRS_CREATE_TRY(dev_alloc(bb, &d.x_proj_t, (size_t)di * xd * esize(bb->dtype)));
            MRS_CREATE_TRY(launch_transpose(bb->stream, bb->dtype, d.x_proj_t, d.x_proj, di, xd));
            if (bb->tiled || bb->split_xproj) {
                MRS_CREATE_TRY(dev_alloc(bb, &d.x_proj_p, tiled_weight_elems(xd, di) * esize(bb->dtype)));
                MRS_CREATE_TRY(launch_tile_weight(bb->stream, bb->dtype, d.x_proj_p, d.x_proj_t, xd, di));
            }
        }
        // a_neg = -exp(a_log) once at load (exp_negate, src/mamba_ssm/gpu/inference.rs:266-282)
        MRS_CREATE_TRY(dev_alloc(bb, (void **)&d.a_neg, (size_t)di * ds * 4));
        { hipError_t e = hipMemcpyAsync(stage, src.a_log, (size_t)di * ds * 4, hipMemcpyHostToDevice, bb->stream);
          if (e != hipSuccess) { mrs_backbone_destroy(bb); return fail(MRS_E_HIP, "a_log upload: %s", hipGetErrorString(e)); } }
        hipLaunchKernelGGL(exp_negate_k, dim3((unsigned)(((size_t)di * ds + 255) / 256)), dim3(256), 0, bb->stream, d.a_neg, stage, (int64_t)di * ds);
        MRS_CREATE_TRY(mrs_a_neg_is_s4d_real(bb->stream, flag, d.a_neg, di, ds));
        int hflag = 0;
        { hipError_t e = hipMemcpyAsync(&hflag, flag, sizeof(int), hipMemcpyDeviceToHost, bb->stream);
          if (e == hipSuccess) e = hipStreamSynchronize(bb->stream);
          if (e != hipSuccess) { mrs_backbone_destroy(bb); return fail(MRS_E_HIP, "s4d flag readback: %s", hipGetErrorString(e)); } }
        d.s4d = hflag;
    }
    MRS_CREATE_TRY(upload_f32(bb, &bb->norm_f, w->norm_f_weight, dm));
    {
        // small f32 models: a step is one launch (MRS_DECODE_NO_TINY=1 keeps the kernel chains)
        const char *e = getenv("MRS_DECODE_NO_TINY");
        if (!(e && atoi(e) != 0) && tiny_step_ok(dtype, input_dim, dm, di, ds, dc, dr, xd) && (!identity || input_dim == dm)) {
            std::vector<TinyStepLayer> tl((size_t)L);
            for (int l = 0; l < L; l++) {
                const LayerDev &d = bb->layers[l];
                tl[(size_t)l] = {d.norm_w, (const float *)d.in_proj, d.conv_w, d.conv_b, (const float *)d.x_proj, (const float *)d.dt_w, d.dt_b, d.a_neg,
                                 d.D, (const float *)d.out_proj};
            }
            MRS_CREATE_TRY(dev_alloc(bb, (void **)&bb->tiny_layers, (size_t)L * sizeof(TinyStepLayer)));
            hipError_t he = hipMemcpyAsync(bb->tiny_layers, tl.data(), (size_t)L * sizeof(TinyStepLayer), hipMemcpyHostToDevice, bb->stream);
            if (he == hipSuccess) he = hipStreamSynchronize(bb->stream);   // tl leaves scope below
            if (he != hipSuccess) { mrs_backbone_destroy(bb); return fail(MRS_E_HIP, "layer table upload: %s", hipGetErrorString(he)); }
        }
    }
    MRS_CREATE_TRY(dev_alloc(bb, (void **)&bb->conv_state, (size_t)L * batch * di * dc * 4));
    MRS_CREATE_TRY(dev_alloc(bb, (void **)&bb->ssm_state, (size_t)L * batch * di * ds * 4));
    MRS_CREATE_TRY(dev_alloc(bb, (void **)&bb->d_input, (size_t)batch * input_dim * 4));
    MRS_CREATE_TRY(dev_alloc(bb, (void **)&bb->temporal, (size_t)batch * dm * 4));
    MRS_CREATE_TRY(dev_alloc(bb, &bb->temporal_t, (size_t)batch * dm * esize(dtype)));
    MRS_CREATE_TRY(alloc_scratch(bb, &bb->step_s, batch, 1));
    MRS_CREATE_TRY(mrs_backbone_reset(bb));
    { hipError_t e = hipStreamSynchronize(bb->stream);
      if (e != hipSuccess) { mrs_backbone_destroy(bb); return fail(MRS_E_HIP, "create sync: %s", hipGetErrorString(e)); } }
#undef MRS_CREATE_TRY
    *out = bb;
    return MRS_OK;
}

extern "C" void mrs_backbone_destroy(mrs_backbone *bb) {
    if (!bb) return;
    hipSetDevice(bb->device);
    if (bb->stream) hipStreamSynchronize(bb->stream);
    if (bb->graph_exec) hipGraphExecDestroy(bb->graph_exec);
    if (bb->graph) hipGraphDestroy(bb->graph);
    for (void *p : bb->allocs) hipFree(p);
    for (void *p : bb->prefill_allocs) hipFree(p);
    gemm_tuner_destroy(bb->tuner);
    if (bb->blas) rocblas_destroy_handle(bb->blas);
    if (bb->stream) hipStreamDestroy(bb->stream);
    delete bb;
}

extern "C" int mrs_backbone_reset(mrs_backbone *bb) {
    if (!bb) return fail(MRS_E_NULL, "mrs_backbone_reset: null engine");
    const size_t L = bb->cfg.n_layers, B = bb->batch;
    MRS_HIP(hipMemsetAsync(bb->conv_state, 0, L * B * bb->di * bb->cfg.d_conv * 4, bb->stream));
    MRS_HIP(hipMemsetAsync(bb->ssm_state, 0, L * B * bb->di * bb->cfg.d_state * 4, bb->stream));
    return MRS_OK;
}

static int step_body(mrs_backbone *bb) {
    if (bb->tiny_layers) {
        TinyStepArgs a = {};
        a.layers = bb->tiny_layers; a.input = bb->d_input;
        a.in_w = bb->identity_proj ? nullptr : bb->input_proj_w; a.in_b = bb->identity_proj ? nullptr : bb->input_proj_b;
        a.norm_f = bb->norm_f; a.conv_state = bb->conv_state; a.ssm_state = bb->ssm_state; a.temporal = bb->temporal;
        a.eps = bb->cfg.rms_norm_eps; a.n_layers = bb->cfg.n_layers; a.batch = bb->batch; a.input_dim = bb->input_dim;
        a.dm = bb->cfg.d_model; a.di = bb->di; a.ds = bb->cfg.d_state; a.dc = bb->cfg.d_conv; a.dr = bb->dr; a.xd = bb->xd;
        return launch_tiny_step(bb->stream, a);
    }
    // identity projection on the own-GEMM chain: the first layer's prenorm kernel reads the input and writes the
    // residual stream itself, so no copy is needed
    bb->step_src = (bb->identity_proj && bb->skinny) ? bb->d_input : nullptr;
    if (!bb->step_src) MRS_TRY(project_input(bb, bb->step_s.residual, bb->d_input, bb->batch));
    return run_layers(bb, &bb->step_s, 1);
}

extern "C" int mrs_backbone_step_gpu_only(mrs_backbone *bb) {
    if (!bb) return fail(MRS_E_NULL, "mrs_backbone_step_gpu_only: null engine");
    if (bb->graph_ready) { MRS_HIP(hipGraphLaunch(bb->graph_exec, bb->stream)); return MRS_OK; }
    return step_body(bb);
}

extern "C" int mrs_backbone_step(mrs_backbone *bb, const float *input, float *output) {
    if (!bb || !input || !output) return fail(MRS_E_NULL, "mrs_backbone_step: null pointer");
    MRS_HIP(hipMemcpyAsync(bb->d_input, input, (size_t)bb->batch * bb->input_dim * 4, hipMemcpyHostToDevice, bb->stream));
    MRS_TRY(mrs_backbone_step_gpu_only(bb));
    MRS_HIP(hipMemcpyAsync(output, bb->temporal, (size_t)bb->batch * bb->cfg.d_model * 4, hipMemcpyDeviceToHost, bb->stream));
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}

// One eager warm step (library handles pick their kernels), reset, then capture the step body
// (src/mamba_ssm/gpu/inference.rs:1608-1630, graph_capture.rs:32-66).  The capture is always ended on error.
extern "C" int mrs_backbone_capture_graph(mrs_backbone *bb) {
    if (!bb) return fail(MRS_E_NULL, "mrs_backbone_capture_graph: null engine");
    if (bb->graph_ready) return MRS_OK;
    // warm step on a copy of the state: save, run, restore
    const size_t L = bb->cfg.n_layers, B = bb->batch;
    const size_t cb = L * B * bb->di * bb->cfg.d_conv * 4, sb = L * B * bb->di * bb->cfg.d_state * 4;
    void *save = nullptr;
    MRS_HIP(hipMalloc(&save, cb + sb));
    hipMemcpyAsync(save, bb->conv_state, cb, hipMemcpyDeviceToDevice, bb->stream);
    hipMemcpyAsync((char *)save + cb, bb->ssm_state, sb, hipMemcpyDeviceToDevice, bb->stream);
    int rc = step_body(bb);
    hipMemcpyAsync(bb->conv_state, save, cb, hipMemcpyDeviceToDevice, bb->stream);
    hipMemcpyAsync(bb->ssm_state, (char *)save + cb, sb, hipMemcpyDeviceToDevice, bb->stream);
    hipStreamSynchronize(bb->stream);
    hipFree(save);
    if (rc) return rc;
    MRS_HIP(hipStreamBeginCapture(bb->stream, hipStreamCaptureModeThreadLocal));
    rc = step_body(bb);
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(bb->stream, &g);
    if (rc) { if (g) hipGraphDestroy(g); return rc; }
    if (e != hipSuccess) return fail(MRS_E_HIP, "hipStreamEndCapture: %s", hipGetErrorString(e));
    e = hipGraphInstantiate(&bb->graph_exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) { hipGraphDestroy(g); return fail(MRS_E_HIP, "hipGraphInstantiate: %s", hipGetErrorString(e)); }
    bb->graph = g;
    bb->graph_ready = 1;
    return MRS_OK;
}

// Prefill scratch follows the sequence length of the call, as the reference allocates it per call
// (src/module/gpu_lm.rs:543-551): the buffers are kept while T stays the same and re-made when it changes.
// Not for use while a capture is open on the engine's stream (it allocates and frees).
static void release_prefill_scratch(mrs_backbone *bb) {
    if (bb->stream) hipStreamSynchronize(bb->stream);   // no kernel may still be reading the old buffers
    for (void *p : bb->prefill_allocs) hipFree(p);
    bb->prefill_allocs.clear();
    bb->prefill_s = Scratch();
    bb->prefill_in = nullptr;
}

extern "C" int mrs_backbone_alloc_prefill_scratch(mrs_backbone *bb, int T) {
    if (!bb) return fail(MRS_E_NULL, "mrs_backbone_alloc_prefill_scratch: null engine");
    if (T < 2) return fail(MRS_E_SHAPE, "mrs_backbone_alloc_prefill_scratch: T=%d (prefill needs T >= 2; use step for one token)", T);
    if ((int64_t)bb->batch * T * bb->di > 0x7fffffffLL) return fail(MRS_E_SHAPE, "prefill: batch*T*d_inner exceeds i32");
    if (bb->prefill_s.rows && bb->prefill_s.T == T) return MRS_OK;
    if (bb->prefill_s.rows) release_prefill_scratch(bb);
    const size_t mark = bb->allocs.size();
    int rc = alloc_scratch(bb, &bb->prefill_s, (int64_t)bb->batch * T, T);
    if (!rc) rc = dev_alloc(bb, (void **)&bb->prefill_in, (size_t)bb->batch * T * bb->input_dim * 4);
    bb->prefill_allocs.assign(bb->allocs.begin() + mark, bb->allocs.end());
    bb->allocs.resize(mark);
    if (rc) release_prefill_scratch(bb);
    return rc;
}

extern "C" int mrs_backbone_prefill_device(mrs_backbone *bb, const float *input_dev, int T) {
    if (!bb || !input_dev) return fail(MRS_E_NULL, "mrs_backbone_prefill_device: null pointer");
    MRS_TRY(mrs_backbone_alloc_prefill_scratch(bb, T));
    MRS_TRY(project_input(bb, bb->prefill_s.residual, input_dev, (int64_t)bb->batch * T));
    return run_layers(bb, &bb->prefill_s, T);
}

extern "C" int mrs_backbone_prefill_sequence(mrs_backbone *bb, const float *input, int T, float *output_last) {
    if (!bb || !input) return fail(MRS_E_NULL, "mrs_backbone_prefill_sequence: null pointer");
    MRS_TRY(mrs_backbone_alloc_prefill_scratch(bb, T));
    MRS_HIP(hipMemcpyAsync(bb->prefill_in, input, (size_t)bb->batch * T * bb->input_dim * 4, hipMemcpyHostToDevice, bb->stream));
    MRS_TRY(mrs_backbone_prefill_device(bb, bb->prefill_in, T));
    if (output_last) MRS_HIP(hipMemcpyAsync(output_last, bb->temporal, (size_t)bb->batch * bb->cfg.d_model * 4, hipMemcpyDeviceToHost, bb->stream));
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}

extern "C" void *mrs_backbone_stream(mrs_backbone *bb) { return bb ? (void *)bb->stream : nullptr; }
extern "C" float *mrs_backbone_temporal_ptr(mrs_backbone *bb) { return bb ? bb->temporal : nullptr; }
// the buffer behind temporal_ptr is f32 whatever the storage type (the 16-bit copy the LM head reads is internal)
extern "C" int mrs_backbone_temporal_dtype(mrs_backbone *bb) { return bb ? MRS_F32 : -1; }
extern "C" int mrs_backbone_decode_route(mrs_backbone *bb) {
    if (!bb) return -1;
    return bb->tiny_layers ? MRS_DECODE_ONE_LAUNCH : bb->skinny ? MRS_DECODE_OWN_CHAIN : MRS_DECODE_LIBRARY_CHAIN;
}
extern "C" int mrs_backbone_download_temporal(mrs_backbone *bb, float *out) {
    if (!bb || !out) return fail(MRS_E_NULL, "mrs_backbone_download_temporal: null pointer");
    MRS_HIP(hipMemcpyAsync(out, bb->temporal, (size_t)bb->batch * bb->cfg.d_model * 4, hipMemcpyDeviceToHost, bb->stream));
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}
extern "C" int mrs_backbone_set_gemm_tuning(mrs_backbone *bb, int on) {
    if (!bb) return fail(MRS_E_NULL, "mrs_backbone_set_gemm_tuning: null engine");
    gemm_tuner_enable(bb->tuner, on);
    return MRS_OK;
}
extern "C" float *mrs_backbone_input_ptr(mrs_backbone *bb) { return bb ? bb->d_input : nullptr; }
extern "C" float *mrs_backbone_prefill_input_ptr(mrs_backbone *bb) { return bb ? bb->prefill_in : nullptr; }
extern "C" int mrs_backbone_sync(mrs_backbone *bb) {
    if (!bb) return fail(MRS_E_NULL, "mrs_backbone_sync: null engine");
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}

extern "C" int mrs_backbone_state_ptrs(mrs_backbone *bb, int layer, float **conv_state, float **ssm_state) {
    if (!bb) return fail(MRS_E_NULL, "mrs_backbone_state_ptrs: null engine");
    if (layer < 0 || layer >= bb->cfg.n_layers) return fail(MRS_E_SHAPE, "mrs_backbone_state_ptrs: layer %d", layer);
    if (conv_state) *conv_state = bb->conv_state + (size_t)layer * bb->batch * bb->di * bb->cfg.d_conv;
    if (ssm_state) *ssm_state = bb->ssm_state + (size_t)layer * bb->batch * bb->di * bb->cfg.d_state;
    return MRS_OK;
}

extern "C" int mrs_backbone_download_state(mrs_backbone *bb, int layer, float *conv_state, float *ssm_state) {
    float *c, *s;
    MRS_TRY(mrs_backbone_state_ptrs(bb, layer, &c, &s));
    if (conv_state) MRS_HIP(hipMemcpyAsync(conv_state, c, (size_t)bb->batch * bb->di * bb->cfg.d_conv * 4, hipMemcpyDeviceToHost, bb->stream));
    if (ssm_state) MRS_HIP(hipMemcpyAsync(ssm_state, s, (size_t)bb->batch * bb->di * bb->cfg.d_state * 4, hipMemcpyDeviceToHost, bb->stream));
    MRS_HIP(hipStreamSynchronize(bb->stream));
    return MRS_OK;
}

// ---- LM: embedding + tied head + greedy loop, all on device -------------------------------
struct mrs_lm {
    LmHooks eng;        // decode engine (not owned)
    mrs_backbone *bb;   // the same engine when it is a Mamba-1 backbone, else null
    void *hid_t;        // head operand in the storage type when the engine keeps none
    int vocab, vocab_padded, dm, batch, dtype;
    void *embed;        // [vocab_padded, dm] storage dtype (tied lm_head)
    void *head;         // [vocab_padded, dm] storage dtype when the head has weights of its own, else null
    // generate_batch state (allocated on first use)
    GenSlots gen;
    GenDyn *gen_dyn;            // device copy
    GenDyn gen_dyn_host;
    int *gen_ints;              // one allocation behind the int arrays of `gen`
    mrs_sampler *gen_samplers;  // [batch]
    unsigned long long *gen_rng;  // [batch, 4]
    float *gen_work;            // [batch, vocab_padded] penalised / scaled logits
    int gen_prompt_cap, gen_out_cap;
    hipGraph_t gen_graph;
    hipGraphExec_t gen_graph_exec;
    int gen_ready, gen_graph_ready;
    float *logits;      // [batch, vocab_padded] f32
    int *tokens;        // [batch] current token ids on device
    float *arg_v;       // [batch, kArgParts] partial maxima
    int *arg_i;
    std::vector<void *> allocs;
    hipGraph_t graph;
    hipGraphExec_t graph_exec;
    int graph_ready;
};

int mrs::launch_embed_gather(hipStream_t st, int dtype, float *out, const void *embed, const int *tokens, int64_t rows, int dm, int vocab) {
    const int64_t n = rows * dm;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    MRS_DISPATCH_DTYPE(dtype, T_, hipLaunchKernelGGL((embed_gather_kernel<T_>), grid, block, 0, st, out, (const T_ *)embed, tokens, rows, dm, vocab,
                                                     (const int *)nullptr));
    return check_launch("embed_gather_kernel");
}

int mrs_lm_create_from_hooks(mrs_lm **out, const LmHooks &eng, const float *embed, int vocab, const char *fn) {
    if (!out || !eng.self || !embed) return fail(MRS_E_NULL, "%s: null pointer", fn);
    if (!eng.identity_proj) return fail(MRS_E_SHAPE, "%s: the LM feeds embeddings straight into the backbone (identity input_proj)", fn);
    if (vocab < 1) return fail(MRS_E_SHAPE, "%s: vocab=%d", fn, vocab);
    mrs_lm *lm = new (std::nothrow) mrs_lm();
    if (!lm) return fail(MRS_E_HIP, "%s: out of host memory", fn);
    lm->eng = eng; lm->bb = nullptr; lm->hid_t = nullptr;
    lm->vocab = vocab; lm->vocab_padded = (vocab + 63) & ~63;  // src/hf/load.rs:59
    lm->dm = eng.d_model; lm->batch = eng.batch; lm->dtype = eng.dtype; lm->graph_ready = 0; lm->graph = nullptr; lm->graph_exec = nullptr;
    lm->head = nullptr;
    lm->gen_ready = 0; lm->gen_graph_ready = 0; lm->gen_graph = nullptr; lm->gen_graph_exec = nullptr;
    lm->gen_prompt_cap = 0; lm->gen_out_cap = 0; lm->gen_dyn = nullptr; lm->gen_dyn_host = GenDyn{nullptr, nullptr, 0};
    *out = nullptr;
    const size_t es = esize(lm->dtype), ne = (size_t)lm->vocab_padded * lm->dm;
    float *stage = nullptr;
    auto cleanup = [&]() { for (void *p : lm->allocs) hipFree(p); if (stage) hipFree(stage); delete lm; };
#define MRS_LM_HIP(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) { cleanup(); return fail(MRS_E_HIP, "%s: %s", #expr, hipGetErrorString(e_)); } } while (0)
    MRS_LM_HIP(hipMalloc(&lm->embed, ne * es)); lm->allocs.push_back(lm->embed);
    MRS_LM_HIP(hipMalloc((void **)&lm->logits, (size_t)lm->batch * lm->vocab_padded * 4)); lm->allocs.push_back(lm->logits);
    MRS_LM_HIP(hipMalloc((void **)&lm->tokens, (size_t)lm->batch * sizeof(int))); lm->allocs.push_back(lm->tokens);
    MRS_LM_HIP(hipMalloc((void **)&lm->arg_v, (size_t)lm->batch * kArgParts * sizeof(float))); lm->allocs.push_back(lm->arg_v);
    MRS_LM_HIP(hipMalloc((void **)&lm->arg_i, (size_t)lm->batch * kArgParts * sizeof(int))); lm->allocs.push_back(lm->arg_i);
    if (!eng.temporal_t && lm->dtype != MRS_F32) { MRS_LM_HIP(hipMalloc(&lm->hid_t, (size_t)lm->batch * lm->dm * es)); lm->allocs.push_back(lm->hid_t); }
    MRS_LM_HIP(hipMalloc((void **)&stage, ne * 4));
    MRS_LM_HIP(hipMemsetAsync(stage, 0, ne * 4, eng.stream));  // padded rows are zero
    MRS_LM_HIP(hipMemcpyAsync(stage, embed, (size_t)vocab * lm->dm * 4, hipMemcpyHostToDevice, eng.stream));
    const dim3 grid((unsigned)((ne + 255) / 256)), block(256);
    if (lm->dtype == MRS_F32) MRS_LM_HIP(hipMemcpyAsync(lm->embed, stage, ne * 4, hipMemcpyDeviceToDevice, eng.stream));
    else if (lm->dtype == MRS_BF16) hipLaunchKernelGGL((cast_from_f32_kernel<bf16_t>), grid, block, 0, eng.stream, (bf16_t *)lm->embed, stage, (int64_t)ne);
    else hipLaunchKernelGGL((cast_from_f32_kernel<f16_t>), grid, block, 0, eng.stream, (f16_t *)lm->embed, stage, (int64_t)ne);
    MRS_LM_HIP(hipStreamSynchronize(eng.stream));
#undef MRS_LM_HIP
    hipFree(stage);
    *out = lm;
    return MRS_OK;
}

// ---- the Mamba-1 engine behind the LM loop ----
static int m1_hook_step(void *self) { return step_body((mrs_backbone *)self); }
static int m1_hook_reset(void *self) { return mrs_backbone_reset((mrs_backbone *)self); }
static size_t m1_hook_state_bytes(void *self) {
    mrs_backbone *bb = (mrs_backbone *)self;
    const size_t L = bb->cfg.n_layers, B = bb->batch;
    return L * B * bb->di * (size_t)(bb->cfg.d_conv + bb->cfg.d_state) * 4;
}
static int m1_hook_state_copy(void *self, void *buf, int restore) {
    mrs_backbone *bb = (mrs_backbone *)self;
    const size_t L = bb->cfg.n_layers, B = bb->batch;
    const size_t cb = L * B * bb->di * bb->cfg.d_conv * 4, sb = L * B * bb->di * bb->cfg.d_state * 4;
    if (restore) {
        MRS_HIP(hipMemcpyAsync(bb->conv_state, buf, cb, hipMemcpyDeviceToDevice, bb->stream));
        MRS_HIP(hipMemcpyAsync(bb->ssm_state, (char *)buf + cb, sb, hipMemcpyDeviceToDevice, bb->stream));
    } else {
        MRS_HIP(hipMemcpyAsync(buf, bb->conv_state, cb, hipMemcpyDeviceToDevice, bb->stream));
        MRS_HIP(hipMemcpyAsync((char *)buf + cb, bb->ssm_state, sb, hipMemcpyDeviceToDevice, bb->stream));
    }
    return MRS_OK;
}
static int m1_hook_prefill(void *self, const int *dev_tokens, const void *embed, int vocab, int T) {
    mrs_backbone *bb = (mrs_backbone *)self;
    MRS_TRY(mrs_backbone_alloc_prefill_scratch(bb, T));
    MRS_TRY(launch_embed_gather(bb->stream, bb->dtype, bb->prefill_in, embed, dev_tokens, (int64_t)bb->batch * T, bb->cfg.d_model, vocab));
    return mrs_backbone_prefill_device(bb, bb->prefill_in, T);
}
static LmHooks m1_hooks(mrs_backbone *bb) {
    LmHooks h = {};
    h.self = bb; h.batch = bb->batch; h.d_model = bb->cfg.d_model; h.dtype = bb->dtype; h.identity_proj = bb->identity_proj;
    h.stream = bb->stream; h.blas = bb->blas; h.d_input = bb->d_input; h.temporal = bb->temporal;
    h.temporal_t = bb->dtype != MRS_F32 ? bb->temporal_t : nullptr;
    h.step = m1_hook_step; h.reset = m1_hook_reset; h.state_bytes = m1_hook_state_bytes; h.state_copy = m1_hook_state_copy; h.prefill = m1_hook_prefill;
    return h;
}

extern "C" int mrs_lm_create(mrs_lm **out, mrs_backbone *bb, const float *embed, int vocab) {
    if (!out || !bb || !embed) return fail(MRS_E_NULL, "mrs_lm_create: null pointer");
    MRS_TRY(mrs_lm_create_from_hooks(out, m1_hooks(bb), embed, vocab, "mrs_lm_create"));
    (*out)->bb = bb;
    return MRS_OK;
}

// A head with weights of its own (tie_word_embeddings = false): `lm_head` is [d_model, vocab] row-major, the
// layout the reference's loader hands over (src/hf/load.rs:126-141, src/module/gpu_lm.rs:182-250).  It is kept
// as [vocab_padded, d_model] like the embedding table, so the logits GEMM is the same call on another pointer.
extern "C" int mrs_lm_set_untied_head(mrs_lm *lm, const float *lm_head) {
    if (!lm || !lm_head) return fail(MRS_E_NULL, "mrs_lm_set_untied_head: null pointer");
    // both graphs bake the head's table pointer in at capture time
    if (lm->graph_ready || lm->gen_graph_ready)
        return fail(MRS_E_SHAPE, "mrs_lm_set_untied_head: set the head before capturing a graph (decode_step capture or a first generate call)");
    const LmHooks *bb = &lm->eng;
    const size_t es = esize(lm->dtype), ne = (size_t)lm->vocab_padded * lm->dm;
    std::vector<float> host;
    try { host.assign(ne, 0.0f); } catch (...) { return fail(MRS_E_HIP, "mrs_lm_set_untied_head: out of host memory"); }
    for (int d = 0; d < lm->dm; ++d)
        for (int v = 0; v < lm->vocab; ++v) host[(size_t)v * lm->dm + d] = lm_head[(size_t)d * lm->vocab + v];
    float *stage = nullptr;
    void *dst = lm->head;
    if (!dst) { MRS_HIP(hipMalloc(&dst, ne * es)); }
    hipError_t e = hipMalloc((void **)&stage, ne * 4);
    if (e == hipSuccess) e = hipMemcpyAsync(stage, host.data(), ne * 4, hipMemcpyHostToDevice, bb->stream);
    if (e == hipSuccess) {
        const dim3 grid((unsigned)((ne + 255) / 256)), block(256);
        if (lm->dtype == MRS_F32) e = hipMemcpyAsync(dst, stage, ne * 4, hipMemcpyDeviceToDevice, bb->stream);
        else if (lm->dtype == MRS_BF16) hipLaunchKernelGGL((cast_from_f32_kernel<bf16_t>), grid, block, 0, bb->stream, (bf16_t *)dst, stage, (int64_t)ne);
        else hipLaunchKernelGGL((cast_from_f32_kernel<f16_t>), grid, block, 0, bb->stream, (f16_t *)dst, stage, (int64_t)ne);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(bb->stream);
    if (stage) hipFree(stage);
    if (e != hipSuccess) { if (!lm->head) hipFree(dst); return fail(MRS_E_HIP, "mrs_lm_set_untied_head: %s", hipGetErrorString(e)); }
    if (!lm->head) { lm->head = dst; lm->allocs.push_back(dst); }
    return MRS_OK;
}

extern "C" void mrs_lm_destroy(mrs_lm *lm) {
    if (!lm) return;
    hipStreamSynchronize(lm->eng.stream);
    if (lm->graph_exec) hipGraphExecDestroy(lm->graph_exec);
    if (lm->graph) hipGraphDestroy(lm->graph);
    if (lm->gen_graph_exec) hipGraphExecDestroy(lm->gen_graph_exec);
    if (lm->gen_graph) hipGraphDestroy(lm->gen_graph);
    if (lm->gen_dyn_host.prompts) hipFree((void *)lm->gen_dyn_host.prompts);
    if (lm->gen_dyn_host.out) hipFree(lm->gen_dyn_host.out);
    for (void *p : lm->allocs) hipFree(p);
    delete lm;
}

// logits = norm_f(hidden) . table^T, table = the embedding (tied head) or the head's own weights
// (OP_T on the row-major [V, dm] table: src/mamba_ssm/gpu/blas.rs:709-740)
static int lm_logits(mrs_lm *lm) {
    const LmHooks *bb = &lm->eng;
    const int dm = lm->dm, V = lm->vocab_padded, B = lm->batch;
    const float one = 1.0f, zero = 0.0f;
    // the head's operand is the final norm's result in the storage type: the engine's own copy (temporal_t), or a cast
    const void *hid = bb->temporal;
    if (lm->dtype != MRS_F32) {
        hid = bb->temporal_t;
        if (!hid) {
            const int64_t n = (int64_t)B * dm;
            const dim3 grid((unsigned)((n + 255) / 256)), block(256);
            if (lm->dtype == MRS_BF16) hipLaunchKernelGGL((cast_from_f32_kernel<bf16_t>), grid, block, 0, bb->stream, (bf16_t *)lm->hid_t, bb->temporal, n);
            else hipLaunchKernelGGL((cast_from_f32_kernel<f16_t>), grid, block, 0, bb->stream, (f16_t *)lm->hid_t, bb->temporal, n);
            hid = lm->hid_t;
        }
    }
    // f32 tables at one to four rows: the table is already [vocab][d_model], the layout the row-wise route of the
    // library's own GEMM walks (the vendor kernel for this shape moves the 154 MB of a 50k x 768 table at 1.6 TB/s)
    const void *table = lm->head ? lm->head : lm->embed;
    if (lm->dtype == MRS_F32 && skinny_gemm_ok(MRS_F32, B, V, dm, dm, hid, table)) {
        const SkinnyEpi none = {};
        return launch_skinny_gemm(bb->stream, MRS_F32, lm->logits, 1, V, hid, dm, table, B, V, dm, none);
    }
    const rocblas_datatype ht = lm->dtype != MRS_F32 ? blas_type(lm->dtype) : rocblas_datatype_f32_r;
    MRS_BLAS(rocblas_gemm_ex((rocblas_handle)bb->blas, rocblas_operation_transpose, rocblas_operation_none, V, B, dm, &one,
                             lm->head ? lm->head : lm->embed, blas_type(lm->dtype), dm, hid, ht, dm, &zero, lm->logits, rocblas_datatype_f32_r, V, lm->logits,
                             rocblas_datatype_f32_r, V, rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0));
    return MRS_OK;
}

static int lm_argmax(mrs_lm *lm) {
    hipStream_t st = lm->eng.stream;
    hipLaunchKernelGGL(argmax_part_kernel, dim3((unsigned)(lm->batch * kArgParts)), dim3(256), 0, st, lm->arg_v, lm->arg_i, lm->logits,
                       lm->vocab, (int64_t)lm->vocab_padded);
    hipLaunchKernelGGL(argmax_final_kernel, dim3((unsigned)lm->batch), dim3(64), 0, st, lm->tokens, lm->arg_v, lm->arg_i);
    return check_launch("argmax kernels");
}

static int lm_decode_body(mrs_lm *lm) {
    const LmHooks *bb = &lm->eng;
    const int64_t n = (int64_t)lm->batch * lm->dm;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    MRS_DISPATCH_DTYPE(lm->dtype, T_, hipLaunchKernelGGL((embed_gather_kernel<T_>), grid, block, 0, bb->stream, bb->d_input,
                                                         (const T_ *)lm->embed, lm->tokens, (int64_t)lm->batch, lm->dm, lm->vocab));
    MRS_TRY(bb->step(bb->self));
    MRS_TRY(lm_logits(lm));
    return lm_argmax(lm);
}

extern "C" int mrs_lm_set_tokens(mrs_lm *lm, const int *tokens) {
    if (!lm || !tokens) return fail(MRS_E_NULL, "mrs_lm_set_tokens: null pointer");
    MRS_HIP(hipMemcpyAsync(lm->tokens, tokens, (size_t)lm->batch * sizeof(int), hipMemcpyHostToDevice, lm->eng.stream));
    return MRS_OK;
}

// One greedy decode step for every batch row, entirely on device: gather embedding of the current
// token, backbone step, tied head, argmax -> next token (left in the device token buffer).
extern "C" int mrs_lm_decode_step(mrs_lm *lm) {
    if (!lm) return fail(MRS_E_NULL, "mrs_lm_decode_step: null engine");
    if (lm->graph_ready) { MRS_HIP(hipGraphLaunch(lm->graph_exec, lm->eng.stream)); return MRS_OK; }
    return lm_decode_body(lm);
}

extern "C" int mrs_lm_capture_graph(mrs_lm *lm) {
    if (!lm) return fail(MRS_E_NULL, "mrs_lm_capture_graph: null engine");
    if (lm->graph_ready) return MRS_OK;
    const LmHooks *bb = &lm->eng;
    // a warm, eager step (the GEMM library settles its choices), with the recurrent state and the tokens put back after it
    const size_t sbytes = bb->state_bytes(bb->self), tb = (size_t)lm->batch * sizeof(int);
    void *save = nullptr;
    MRS_HIP(hipMalloc(&save, sbytes + tb));
    int rc = bb->state_copy(bb->self, save, 0);
    hipMemcpyAsync((char *)save + sbytes, lm->tokens, tb, hipMemcpyDeviceToDevice, bb->stream);
    if (!rc) rc = lm_decode_body(lm);
    if (!rc) rc = bb->state_copy(bb->self, save, 1);
    hipMemcpyAsync(lm->tokens, (char *)save + sbytes, tb, hipMemcpyDeviceToDevice, bb->stream);
    hipStreamSynchronize(bb->stream);
    hipFree(save);
    if (rc) return rc;
    MRS_HIP(hipStreamBeginCapture(bb->stream, hipStreamCaptureModeThreadLocal));
    rc = lm_decode_body(lm);
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(bb->stream, &g);
    if (rc) { if (g) hipGraphDestroy(g); return rc; }
    if (e != hipSuccess) return fail(MRS_E_HIP, "hipStreamEndCapture: %s", hipGetErrorString(e));
    e = hipGraphInstantiate(&lm->graph_exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) { hipGraphDestroy(g); return fail(MRS_E_HIP, "hipGraphInstantiate: %s", hipGetErrorString(e)); }
    lm->graph = g; lm->graph_ready = 1;
    return MRS_OK;
}

extern "C" int mrs_lm_get_tokens(mrs_lm *lm, int *tokens) {
    if (!lm || !tokens) return fail(MRS_E_NULL, "mrs_lm_get_tokens: null pointer");
    MRS_HIP(hipMemcpyAsync(tokens, lm->tokens, (size_t)lm->batch * sizeof(int), hipMemcpyDeviceToHost, lm->eng.stream));
    MRS_HIP(hipStreamSynchronize(lm->eng.stream));
    return MRS_OK;
}

extern "C" int mrs_lm_last_logits(mrs_lm *lm, float *logits) {
    if (!lm || !logits) return fail(MRS_E_NULL, "mrs_lm_last_logits: null pointer");
    MRS_HIP(hipMemcpy2DAsync(logits, (size_t)lm->vocab * 4, lm->logits, (size_t)lm->vocab_padded * 4, (size_t)lm->vocab * 4, lm->batch,
                             hipMemcpyDeviceToHost, lm->eng.stream));
    MRS_HIP(hipStreamSynchronize(lm->eng.stream));
    return MRS_OK;
}

// Prefill helper for the LM: token ids [batch, T] (host) -> embeddings on device -> backbone prefill,
// then the head on the last position; the greedy next token of every row is left in the token buffer.
// prefill_bb: a Mamba-1 engine (the LM's own or another one with the prefill batch), or null = the LM's own engine.
extern "C" int mrs_lm_prefill(mrs_lm *lm, mrs_backbone *prefill_bb, const int *tokens, int T) {
    if (!lm || !tokens) return fail(MRS_E_NULL, "mrs_lm_prefill: null pointer");
    if (T < 1) return fail(MRS_E_SHAPE, "mrs_lm_prefill: T=%d", T);
    const bool own = !prefill_bb || prefill_bb == lm->bb;
    LmHooks other = {};
    if (!own) {
        if (prefill_bb->cfg.d_model != lm->dm || prefill_bb->dtype != lm->dtype || !prefill_bb->identity_proj)
            return fail(MRS_E_SHAPE, "mrs_lm_prefill: prefill engine does not match the LM");
        other = m1_hooks(prefill_bb);
    }
    const LmHooks *eng = own ? &lm->eng : &other;
    const int64_t rows = (int64_t)eng->batch * T;
    int *dtok = nullptr;
    MRS_HIP(hipMalloc((void **)&dtok, rows * sizeof(int)));
    hipMemcpyAsync(dtok, tokens, rows * sizeof(int), hipMemcpyHostToDevice, eng->stream);
    int rc = eng->prefill(eng->self, dtok, lm->embed, lm->vocab, T);
    if (!rc && own) {
        rc = lm_logits(lm);
        if (!rc) rc = lm_argmax(lm);
    }
    hipStreamSynchronize(eng->stream);
    hipFree(dtok);
    return rc;
}

// ---- batched generation ------------------------------------------------------------------------------------

static int gen_alloc(mrs_lm *lm) {
    if (lm->gen_ready) return MRS_OK;
    const size_t B = lm->batch;
    const size_t n_int = B * (10 + kMaxEos) + 1;
    MRS_HIP(hipMalloc((void **)&lm->gen_ints, n_int * sizeof(int))); lm->allocs.push_back(lm->gen_ints);
    int *p = lm->gen_ints;
    GenSlots &g = lm->gen;
    g.prompt_off = p; p += B; g.prompt_len = p; p += B; g.prompt_pos = p; p += B; g.finished = p; p += B; g.active = p; p += B;
    g.max_tokens = p; p += B; g.n_eos = p; p += B; g.out_len = p; p += B; g.sampled = p; p += B; p += B /* spare */;
    g.eos = p; p += B * kMaxEos; g.n_running = p;
    MRS_HIP(hipMalloc((void **)&g.seen, B * lm->vocab * sizeof(unsigned))); lm->allocs.push_back(g.seen);
    MRS_HIP(hipMalloc((void **)&lm->gen_samplers, B * sizeof(mrs_sampler))); lm->allocs.push_back(lm->gen_samplers);
    MRS_HIP(hipMalloc((void **)&lm->gen_rng, B * 4 * sizeof(unsigned long long))); lm->allocs.push_back(lm->gen_rng);
    MRS_HIP(hipMalloc((void **)&lm->gen_work, B * lm->vocab_padded * sizeof(float))); lm->allocs.push_back(lm->gen_work);
    MRS_HIP(hipMalloc((void **)&lm->gen_dyn, sizeof(GenDyn))); lm->allocs.push_back(lm->gen_dyn);
    lm->gen_ready = 1;
    return MRS_OK;
}

// sample the active slots from the current logits, then advance every slot
static int gen_pick(mrs_lm *lm) {
    hipStream_t st = lm->eng.stream;
    MRS_TRY(launch_sample_rows(st, lm->gen.sampled, lm->logits, lm->gen_work, lm->vocab_padded, lm->batch, lm->vocab, lm->gen_samplers,
                               lm->gen.seen, lm->gen_rng, lm->gen.active));
    hipLaunchKernelGGL(gen_advance_kernel, dim3(1), dim3(1024), 0, st, lm->gen, lm->gen_dyn, lm->tokens, lm->batch, lm->vocab);
    return check_launch("gen_advance_kernel");
}

// gather the slots' current tokens (zeros for finished slots), one backbone step, head
static int gen_forward(mrs_lm *lm) {
    const LmHooks *bb = &lm->eng;
    const int64_t n = (int64_t)lm->batch * lm->dm;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    MRS_DISPATCH_DTYPE(lm->dtype, T_, hipLaunchKernelGGL((embed_gather_kernel<T_>), grid, block, 0, bb->stream, bb->d_input,
                                                         (const T_ *)lm->embed, lm->tokens, (int64_t)lm->batch, lm->dm, lm->vocab,
                                                         (const int *)lm->gen.finished));
    MRS_TRY(bb->step(bb->self));
    return lm_logits(lm);
}

// The generation loop behind mrs_lm_generate_batch and mrs_lm_generate_streaming.  With a callback (batch 1) the host
// looks at the slot after every step instead of every 16th and hands each new token over as it appears.
static int gen_run(mrs_lm *lm, const int *prompts, const int *prompt_lens, const mrs_sample_params *params, int seen_includes_prompt,
                   int *out_tokens, int out_stride, int *out_lens, mrs_token_callback cb, void *user) {
    if (!lm || !prompt_lens || !params || !out_tokens || !out_lens) return fail(MRS_E_NULL, "mrs_lm_generate_batch: null pointer");
    const LmHooks *bb = &lm->eng;
    hipStream_t st = bb->stream;
    const int B = lm->batch;
    int64_t total = 0;
    int max_prompt = 0, max_tokens = 0;
    for (int i = 0; i < B; i++) {
        if (prompt_lens[i] < 0 || params[i].max_tokens < 0 || params[i].n_eos < 0 || params[i].n_eos > kMaxEos ||
            (params[i].n_eos > 0 && !params[i].eos_token_ids))
            return fail(MRS_E_SHAPE, "mrs_lm_generate_batch: slot %d: prompt_len=%d max_tokens=%d n_eos=%d (at most %d)", i, prompt_lens[i],
                        params[i].max_tokens, params[i].n_eos, kMaxEos);
        if (params[i].max_tokens > out_stride)
            return fail(MRS_E_SHAPE, "mrs_lm_generate_batch: slot %d: max_tokens=%d exceeds out_stride=%d", i, params[i].max_tokens, out_stride);
        total += prompt_lens[i];
        max_prompt = std::max(max_prompt, prompt_lens[i]);
        max_tokens = std::max(max_tokens, params[i].max_tokens);
    }
    if (total > 0 && !prompts) return fail(MRS_E_NULL, "mrs_lm_generate_batch: null prompts");
    if (total > (int64_t)1 << 30) return fail(MRS_E_SHAPE, "mrs_lm_generate_batch: %lld prompt tokens", (long long)total);
    MRS_TRY(gen_alloc(lm));
    // buffers that follow the call's sizes
    if (total > lm->gen_prompt_cap) {
        if (lm->gen_dyn_host.prompts) hipFree((void *)lm->gen_dyn_host.prompts);
        lm->gen_dyn_host.prompts = nullptr; lm->gen_prompt_cap = 0;
        int *p = nullptr;
        MRS_HIP(hipMalloc((void **)&p, (size_t)total * sizeof(int)));
        lm->gen_dyn_host.prompts = p; lm->gen_prompt_cap = (int)total;
    }
    const int64_t out_need = (int64_t)B * std::max(max_tokens, 1);
    if (out_need > lm->gen_out_cap) {
        if (lm->gen_dyn_host.out) hipFree(lm->gen_dyn_host.out);
        lm->gen_dyn_host.out = nullptr; lm->gen_out_cap = 0;
        MRS_HIP(hipMalloc((void **)&lm->gen_dyn_host.out, (size_t)out_need * sizeof(int)));
        lm->gen_out_cap = (int)out_need;
    }
    lm->gen_dyn_host.out_stride = std::max(max_tokens, 1);
    // host-side initial state (gpu_lm.rs:404-430): the first prompt token is the first input; empty prompts are finished
    std::vector<int> h((size_t)B * (10 + kMaxEos) + 1, 0);
    int *off = h.data(), *len = off + B, *pos = len + B, *fin = pos + B, *act = fin + B, *mx = act + B, *neos = mx + B, *olen = neos + B,
        *eos = olen + 3 * B, *nrun = eos + (size_t)B * kMaxEos;
    std::vector<int> first(B, 0);
    std::vector<mrs_sampler> samplers(B);
    std::vector<unsigned long long> rng((size_t)B * 4);
    const bool prefill_route = seen_includes_prompt && B == 1 && prompt_lens[0] >= 256;   // PREFILL_PARALLEL_THRESHOLD, gpu_lm.rs:48
    int64_t o = 0;
    int running = 0;
    for (int i = 0; i < B; i++) {
        off[i] = (int)o; len[i] = prompt_lens[i]; o += prompt_lens[i];
        fin[i] = prompt_lens[i] == 0;
        pos[i] = fin[i] ? 0 : (prefill_route ? len[i] : 1);
        act[i] = !fin[i] && pos[i] >= len[i];
        first[i] = fin[i] ? 0 : prompts[off[i]];
        mx[i] = params[i].max_tokens; neos[i] = params[i].n_eos;
        for (int e = 0; e < params[i].n_eos; e++) eos[(size_t)i * kMaxEos + e] = params[i].eos_token_ids[e];
        samplers[i] = params[i].sampler;
        mrs_xoshiro_seed(params[i].seed, &rng[(size_t)i * 4]);
        running += !fin[i];
    }
    *nrun = running;
    MRS_HIP(hipMemcpyAsync(lm->gen_ints, h.data(), h.size() * sizeof(int), hipMemcpyHostToDevice, st));
    MRS_HIP(hipMemcpyAsync(lm->gen_samplers, samplers.data(), samplers.size() * sizeof(mrs_sampler), hipMemcpyHostToDevice, st));
    MRS_HIP(hipMemcpyAsync(lm->gen_rng, rng.data(), rng.size() * sizeof(unsigned long long), hipMemcpyHostToDevice, st));
    MRS_HIP(hipMemcpyAsync(lm->gen_dyn, &lm->gen_dyn_host, sizeof(GenDyn), hipMemcpyHostToDevice, st));
    if (total > 0) MRS_HIP(hipMemcpyAsync((void *)lm->gen_dyn_host.prompts, prompts, (size_t)total * sizeof(int), hipMemcpyHostToDevice, st));
    MRS_HIP(hipMemcpyAsync(lm->tokens, first.data(), (size_t)B * sizeof(int), hipMemcpyHostToDevice, st));
    MRS_HIP(hipMemsetAsync(lm->gen.seen, 0, (size_t)B * lm->vocab * sizeof(unsigned), st));
    MRS_HIP(hipStreamSynchronize(st));   // the staging vectors above go out of use here
    if (seen_includes_prompt && max_prompt > 0)
        hipLaunchKernelGGL(gen_seen_prompt_kernel, dim3((unsigned)std::min(64, (max_prompt + 255) / 256), (unsigned)B), dim3(256), 0, st, lm->gen,
                           lm->gen_dyn, B, lm->vocab);
    MRS_TRY(bb->reset(bb->self));
    int steps = max_prompt + max_tokens;   // gpu_lm.rs:432
    if (prefill_route && running) {
        MRS_TRY(mrs_lm_prefill(lm, nullptr, prompts, prompt_lens[0]));   // state after the prompt, logits of its last position
        MRS_TRY(gen_pick(lm));
        steps = max_tokens;
    }
    int done = 0, emitted = 0;
    bool stopped = false;
    for (int s = 0; s < steps && running > 0; s++) {
        if (lm->gen_graph_ready) {
            MRS_HIP(hipGraphLaunch(lm->gen_graph_exec, st));
        } else if (s == 1) {
            // the first step ran eagerly (the GEMM library settles its choices); capture the step now and replay it from here on
            MRS_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
            int rc = gen_forward(lm);
            if (!rc) rc = gen_pick(lm);
            hipGraph_t gph = nullptr;
            hipError_t e = hipStreamEndCapture(st, &gph);
            if (rc) { if (gph) hipGraphDestroy(gph); return rc; }
            if (e != hipSuccess) return fail(MRS_E_HIP, "hipStreamEndCapture: %s", hipGetErrorString(e));
            e = hipGraphInstantiate(&lm->gen_graph_exec, gph, nullptr, nullptr, 0);
            if (e != hipSuccess) { hipGraphDestroy(gph); return fail(MRS_E_HIP, "hipGraphInstantiate: %s", hipGetErrorString(e)); }
            lm->gen_graph = gph; lm->gen_graph_ready = 1;
            MRS_HIP(hipGraphLaunch(lm->gen_graph_exec, st));
        } else {
            MRS_TRY(gen_forward(lm));
            MRS_TRY(gen_pick(lm));
        }
        if (cb) {
            // streaming (one slot): the slot's output length and the token at the next unread position, every step
            int olen_now = 0, tok = 0;
            MRS_HIP(hipMemcpyAsync(&running, lm->gen.n_running, sizeof(int), hipMemcpyDeviceToHost, st));
            MRS_HIP(hipMemcpyAsync(&olen_now, lm->gen.out_len, sizeof(int), hipMemcpyDeviceToHost, st));
            if (emitted < lm->gen_dyn_host.out_stride)
                MRS_HIP(hipMemcpyAsync(&tok, lm->gen_dyn_host.out + emitted, sizeof(int), hipMemcpyDeviceToHost, st));
            MRS_HIP(hipStreamSynchronize(st));
            ++done;
            if (olen_now > emitted) {
                emitted++;
                if (cb(tok, user) != 0) { stopped = true; break; }   // the caller has seen enough
            }
        } else if (++done % 16 == 0 || s + 1 == steps) {   // the only host round trip of the loop: is anyone still running?
            MRS_HIP(hipMemcpyAsync(&running, lm->gen.n_running, sizeof(int), hipMemcpyDeviceToHost, st));
            MRS_HIP(hipStreamSynchronize(st));
        }
    }
    MRS_HIP(hipMemcpyAsync(out_lens, lm->gen.out_len, (size_t)B * sizeof(int), hipMemcpyDeviceToHost, st));
    MRS_HIP(hipMemcpy2DAsync(out_tokens, (size_t)out_stride * sizeof(int), lm->gen_dyn_host.out, (size_t)lm->gen_dyn_host.out_stride * sizeof(int),
                             (size_t)std::min(out_stride, lm->gen_dyn_host.out_stride) * sizeof(int), B, hipMemcpyDeviceToHost, st));
    MRS_HIP(hipStreamSynchronize(st));
    if (cb) {
        // stopped by the callback: what was handed over; else whatever the loop has not handed over yet (after a
        // prefilled prompt the first token exists before the first step, so the hand-over runs one step behind)
        if (stopped) out_lens[0] = emitted;
        for (; !stopped && emitted < out_lens[0]; emitted++)
            if (cb(out_tokens[emitted], user) != 0) { out_lens[0] = emitted + 1; break; }
    }
    return MRS_OK;
}

extern "C" int mrs_lm_generate_batch(mrs_lm *lm, const int *prompts, const int *prompt_lens, const mrs_sample_params *params,
                                     int seen_includes_prompt, int *out_tokens, int out_stride, int *out_lens) {
    return gen_run(lm, prompts, prompt_lens, params, seen_includes_prompt, out_tokens, out_stride, out_lens, nullptr, nullptr);
}

extern "C" int mrs_lm_generate_streaming(mrs_lm *lm, const int *prompt, int prompt_len, const mrs_sample_params *params,
                                         mrs_token_callback cb, void *user) {
    if (!lm || !params || !cb) return fail(MRS_E_NULL, "mrs_lm_generate_streaming: null pointer");
    if (lm->batch != 1) return fail(MRS_E_SHAPE, "mrs_lm_generate_streaming: batch=%d (a batch-1 engine; mrs_lm_generate_batch for more)", lm->batch);
    if (params->max_tokens < 0) return fail(MRS_E_SHAPE, "mrs_lm_generate_streaming: max_tokens=%d", params->max_tokens);
    std::vector<int> out((size_t)std::max(params->max_tokens, 1));
    int n = 0;
    return gen_run(lm, prompt, &prompt_len, params, 1, out.data(), (int)out.size(), &n, cb, user);
}
