/*
 * mamba_hip.h -- C ABI of libmamba_hip.so: the MI355X (gfx950) Mamba inference
 * hot path.  Plain pointers and sizes only; every device pointer is a HIP
 * device address, `stream` is a hipStream_t passed as void* (NULL = the null
 * stream).  All entry points are stream-ordered, never allocate, never
 * synchronise (unless stated) and return 0 on success or a negative MRS_E_*
 * code, with a message available from mrs_last_error() on the calling thread.
 *
 * Each declaration names the reference interface it replaces
 * (silvermpx/mamba-rs v0.5.3, paths relative to that repository).  The
 * reference looks its kernels up by name in one NVRTC module and launches them
 * with positional raw-pointer/int arguments (src/mamba_ssm/gpu/kernels.rs:547-700);
 * the argument order of those launch sites is kept, with `stream` and `dtype`
 * put in front.
 */
#ifndef MAMBA_HIP_H
#define MAMBA_HIP_H

#include <stddef.h>
#include <stdint.h>

/* Exported symbol marker: the library is built with hidden visibility. */
#define MRS_API __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

/* Activation storage type.  Values follow the declaration order of the
 * reference's WeightDtype enum (src/mamba_ssm/gpu/dtype.rs:12-28).  Compute is
 * always f32; SSM state, conv state, a_neg, D, biases stay f32. */
typedef enum { MRS_F32 = 0, MRS_F16 = 1, MRS_BF16 = 2 } mrs_dtype;

/* Scan route request, mirrors ScanMode (src/config.rs:6-18). */
typedef enum { MRS_SCAN_SEQUENTIAL = 0, MRS_SCAN_PARALLEL = 1, MRS_SCAN_AUTO = 2 } mrs_scan_mode;

enum {
    MRS_OK = 0,
    MRS_E_NULL = -1,        /* a required pointer is NULL */
    MRS_E_SHAPE = -2,       /* unsupported or inconsistent shape */
    MRS_E_DTYPE = -3,       /* dtype not one of mrs_dtype */
    MRS_E_WORKSPACE = -4,   /* workspace missing or too small */
    MRS_E_ALIGN = -5,       /* a pointer breaks the stated alignment */
    MRS_E_HIP = -6          /* the HIP runtime reported an error at launch */
};

/* Flags for mrs_ssm_scan_fwd_ex. */
enum {
    MRS_GATE_NONE = 0,
    MRS_GATE_PREACT = 1u << 0, /* gate holds silu(z) already: y *= gate (kernels/mamba_ssm.cu:220-222) */
    MRS_GATE_SILU = 1u << 1,   /* gate holds raw z: y *= z*sigmoid(z) (split_gate_silu + elementwise_mul fused) */
    MRS_A_S4D_REAL = 1u << 2,  /* caller asserts a_neg[d,n] = (n+1)*a_neg[d,0] to 4 ulp; see mrs_a_neg_is_s4d_real */
    MRS_FORCE_SEQUENTIAL = 1u << 3, /* ignore the T-split route */
    MRS_FORCE_PARALLEL = 1u << 4,   /* use the T-split route even for short T, and its one-launch form at any size */
    MRS_SCAN_FLAGS_ZERO = 1u << 5,  /* T-split route: the caller vouches that the first mrs_ssm_scan_flag_bytes() bytes of
                                       the workspace were zero before the first call and that nothing but this entry
                                       point has written there since; saves the small kernel that clears them */
    MRS_SCAN_TWO_LAUNCHES = 1u << 6 /* T-split route as two launches (no wave waits for another; also MRS_SCAN_TWO_LAUNCHES=1
                                       in the environment) */
};

/* Library version (major*10000 + minor*100 + patch) and the last error text of
 * the calling thread ("" if none). */
MRS_API int mrs_version(void);
MRS_API const char *mrs_last_error(void);

/* ScanMode::use_parallel (src/config.rs:28-37): 1 if the parallel route is
 * chosen for (mode, seq_len, d_state).  d_state > 64 always answers 1. */
MRS_API int mrs_scan_use_parallel(int mode, int64_t seq_len, int64_t d_state);

/* exp_negate kernel (kernels/elementwise.cu:140-146; called from
 * src/mamba_ssm/gpu/inference.rs:266-282): a_neg[i] = -exp(a_log[i]), n floats. */
MRS_API int mrs_exp_negate(void *stream, float *a_neg, const float *a_log, int64_t n);

/* Writes 1 to *flag_out (a device int) if |a_neg[d,n] - (n+1)*a_neg[d,0]| <=
 * 2^-21 |a_neg[d,n]| (4 ulp) for every d,n -- the S4D-real initialisation
 * a_log = log(1..=d_state) (src/weights.rs:143-148), whose a_neg = -exp(a_log)
 * is (n+1) to within an ulp or two -- else 0.  No counterpart in the reference;
 * it licenses MRS_A_S4D_REAL, under which exp(delta*a_neg[d,n]) is formed as
 * exp(delta*a_neg[d,0])^(n+1) (relative deviation <= |delta*a_neg| * 5e-7). */
MRS_API int mrs_a_neg_is_s4d_real(void *stream, int *flag_out, const float *a_neg, int d_inner, int d_state);

/* ---- Mamba-1 selective scan, full sequence --------------------------------
 * Replaces ssm_parallel_scan_fwd_nosave_{f32,bf16,f16}
 * (kernels/mamba_ssm_parallel.cu:544-765, 969-1145) and
 * ssm_burnin_forward_nosave_{..} (kernels/mamba_ssm.cu:304-400); launch sites
 * src/mamba_ssm/gpu/prefill.rs:512-549, 910-956, argument order
 * h, y, delta, u, B, C, a_neg, D, batch, T, d_inner, d_state.
 *   h      [batch, d_inner, d_state] f32, read and overwritten with the final state
 *   y      [batch, T, d_inner]       dtype
 *   delta,u[batch, T, d_inner]       dtype (delta after softplus)
 *   B, C   [batch, T, d_state]       dtype
 *   a_neg  [d_inner, d_state] f32,  D [d_inner] f32
 * d_state in 1..=256, T >= 1.  This symbol keeps the reference's argument list, which has no room for a workspace, and
 * therefore always takes the sequential kernel (one wave per 64 channels of a batch row: about 0.9 ms at
 * 8 x 2048 x 1536 where the T-split route takes 0.1 ms).  A caller replacing the *parallel* launch site
 * (src/mamba_ssm/gpu/prefill.rs:910-933) should bind mrs_ssm_scan_fwd_ex (workspace) or mrs_ssm_scan_fwd_static
 * (none) instead. */
MRS_API int mrs_ssm_scan_fwd(void *stream, int dtype, float *h, void *y, const void *delta, const void *u,
                     const void *B, const void *C, const float *a_neg, const float *D,
                     int batch, int T, int d_inner, int d_state);

/* Same scan with the fusions the prefill chain allows:
 *   bc_stride  row stride (elements) of B and C, so both can point into xdbl
 *              [batch*T, xdbl_dim] (replaces gather_bc_cols, kernels/elementwise.cu:291-313)
 *   gate,flags optional gate tensor, [batch*T] rows of gate_stride elements (0 = d_inner), the
 *              first d_inner of each used (replaces elementwise_mul, src/mamba_ssm/gpu/prefill.rs:957-971;
 *              with MRS_GATE_SILU and gate_stride = 2*d_inner it reads the z half of in_proj's
 *              output in place, which also replaces split_gate_silu, kernels/elementwise.cu:172-189)
 *   workspace  mrs_ssm_scan_workspace_bytes() bytes of device memory, 256-byte
 *              aligned; NULL forces the sequential route. */
MRS_API size_t mrs_ssm_scan_workspace_bytes(int batch, int T, int d_inner, int d_state);
/* Where it is the faster form -- MRS_A_S4D_REAL and at least 2048 waves (batch x ceil(d_inner / 64) x chunks) -- the
 * T-split route runs as ONE launch: every wave first summarises its chunk, publishes the summary and waits for the
 * chunks before it (no counterpart in the reference, whose kernel keeps a block per (b, d) and needs no such hand-off).
 * The flags the waves signal with are the first mrs_ssm_scan_flag_bytes(batch, d_inner) bytes of the workspace (256 KB
 * whatever the shape, counted in mrs_ssm_scan_workspace_bytes); they must be zero when the launch starts and are zero
 * again when it ends.  By default a small kernel clears them ahead of every call; a caller that zeroed them once (and
 * lets nothing else write there) passes MRS_SCAN_FLAGS_ZERO and saves that kernel.  MRS_SCAN_TWO_LAUNCHES keeps the
 * two-kernel form, MRS_FORCE_PARALLEL takes the one launch at any size and for any A.  A wave that waits some seconds
 * for another (never seen; it would take a wave that does not get scheduled) writes NaN into its share
 * of y and h rather than spin for ever. */
MRS_API size_t mrs_ssm_scan_flag_bytes(int batch, int d_inner);
MRS_API int mrs_ssm_scan_fwd_ex(void *stream, int dtype, float *h, void *y, const void *delta, const void *u,
                        const void *B, const void *C, int64_t bc_stride, const float *a_neg,
                        const float *D, const void *gate, int64_t gate_stride, unsigned flags,
                        void *workspace, size_t workspace_bytes,
                        int batch, int T, int d_inner, int d_state);

/* mrs_ssm_scan_fwd_ex without the workspace argument, for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose launch site allocates nothing either, because its kernel keeps no chunk summaries in memory).
 * The chunk summaries of the T-split route go to a device buffer the library holds itself -- one
 * MRS_SCAN_STATIC_SCRATCH_BYTES block per GPU, resident until the process ends -- so the call allocates nothing
 * and frees nothing.  Same arguments, routes and results as mrs_ssm_scan_fwd_ex given a workspace of that size.
 *   - A shape with mrs_ssm_scan_workspace_bytes() > MRS_SCAN_STATIC_SCRATCH_BYTES is refused (MRS_E_WORKSPACE);
 *     the benchmark shapes (8 x 2048 x 1536 and 4 x 4096 x 5120, d_state 16) need 13.6 MB and 12.8 MB; only very wide
 *     batches (batch x d_inner above about 120 000 channels) need more.
 *   - The first call on a GPU looks the buffer's address up (hipGetSymbolAddress, no allocation); make that call
 *     outside a graph capture.
 *   - All calls on one GPU share the one buffer: two calls that overlap in time on the same GPU (different
 *     streams, or graphs replayed side by side) race.  Serialise them or use mrs_ssm_scan_fwd_ex. */
#define MRS_SCAN_STATIC_SCRATCH_BYTES (16u << 20)
MRS_API int mrs_ssm_scan_fwd_static(void *stream, int dtype, float *h, void *y, const void *delta, const void *u,
                        const void *B, const void *C, int64_t bc_stride, const float *a_neg,
                        const float *D, const void *gate, int64_t gate_stride, unsigned flags,
                        int batch, int T, int d_inner, int d_state);

/* ---- Mamba-1 selective scan, one step (decode) ------------------------------
 * ssm_step_forward_{..} (kernels/mamba_ssm.cu:26-116; src/mamba_ssm/gpu/inference.rs:669-698):
 * delta,u,y [batch,d_inner]; B,C [batch,d_state]. */
MRS_API int mrs_ssm_step(void *stream, int dtype, float *h, void *y, const void *delta, const void *u,
                 const void *B, const void *C, const float *a_neg, const float *D,
                 int batch, int d_inner, int d_state);

/* ssm_step_forward_gather_gate_{..} (kernels/mamba_ssm.cu:180-227;
 * src/mamba_ssm/gpu/inference.rs:1182-1215): B and C are read from
 * xdbl[b*xdbl_stride + b_offset + n] / [.. + c_offset + n]; y *= gate_silu.
 * gate_silu == NULL gives ssm_step_forward_gather_{..} (kernels/mamba_ssm.cu:126-170). */
MRS_API int mrs_ssm_step_gather_gate(void *stream, int dtype, float *h, void *y, const void *delta,
                             const void *u, const void *xdbl, const void *gate_silu,
                             const float *a_neg, const float *D, int batch, int d_inner, int d_state,
                             int xdbl_stride, int b_offset, int c_offset);

/* ---- causal depthwise conv1d (+SiLU) ----------------------------------------
 * conv1d_step_forward_silu_{..} (kernels/conv1d.cu:85-115;
 * src/mamba_ssm/gpu/inference.rs:1062-1084), order out,state,new_x,weight,bias,batch,d_inner,d_conv.
 *   state [batch,d_inner,d_conv] f32 window, shifted left and updated in place
 *   new_x,out [batch,d_inner] dtype; weight [d_inner,d_conv], bias [d_inner] f32
 * apply_silu = 0 gives conv1d_step_forward_{..} (kernels/conv1d.cu:14-75). d_conv in 1..=8. */
MRS_API int mrs_conv1d_step(void *stream, int dtype, void *out, float *state, const void *new_x,
                    const float *weight, const float *bias, int batch, int d_inner, int d_conv,
                    int apply_silu);

/* conv1d_burnin_forward_nosave_{..} (kernels/conv1d.cu:209-315;
 * src/mamba_ssm/gpu/prefill.rs:417-439, 780-804), order u_out,state,x_branch,weight,bias,batch,T,d_inner,d_conv.
 *   x_branch rows of x_stride elements ([batch*T] rows; x_stride = d_inner for the
 *   reference's split buffer, 2*d_inner to read the x half of in_proj's output in place)
 *   u_out [batch,T,d_inner] dtype, SiLU applied. */
MRS_API int mrs_conv1d_seq_silu(void *stream, int dtype, void *u_out, float *state, const void *x_branch,
                        int64_t x_stride, const float *weight, const float *bias,
                        int batch, int T, int d_inner, int d_conv);

/* ---- Mamba-3 SISO trapezoidal scan --------------------------------------------
 * State of one layer (all f32, mutated in place): ssm_state [batch,nheads,headdim,d_state],
 * k_state [batch,nheads,d_state] (previous K after bias+RoPE), v_state [batch,nheads,headdim]
 * (previous x).  d_inner = nheads*headdim.
 *
 * m3_step_fwd_{..} (kernels/mamba3_ssd.cu:56-215; src/mamba3_siso/gpu/inference.rs:756-784),
 * order ssm,k,v,y,x,k_cur,q_cur,alpha,beta,gamma,D,batch,nh,hd,ds:
 *   x,y [batch,d_inner] dtype; k_cur,q_cur [batch,nheads,d_state] dtype;
 *   alpha,beta,gamma [batch,nheads] f32; D [nheads] f32.
 * headdim <= 1024 and d_state <= 256 (the reference stops at headdim 32, d_state 64). */
MRS_API int mrs_m3_step(void *stream, int dtype, float *ssm_state, float *k_state, float *v_state, void *y,
                        const void *x, const void *k_cur, const void *q_cur, const float *alpha,
                        const float *beta, const float *gamma, const float *D, int batch, int nheads,
                        int headdim, int d_state);

/* m3_burnin_fwd_nosave_{..} (kernels/mamba3_ssd.cu:453-546; src/mamba3_siso/gpu/forward.rs:423-455):
 * the same recurrence over T steps, state carried in and out.
 *   x,y [batch,T,d_inner]; k,q [batch,T,nheads,d_state]; alpha,beta,gamma [batch,T,nheads]. */
MRS_API int mrs_m3_seq_fwd(void *stream, int dtype, float *ssm_state, float *k_state, float *v_state,
                           void *y, const void *x, const void *k, const void *q, const float *alpha,
                           const float *beta, const float *gamma, const float *D, int batch, int T,
                           int nheads, int headdim, int d_state);

/* m3_compute_abg (kernels/mamba3_ops.cu:735-753): alpha = exp(a_val*dt), beta = alpha*dt*(1-trap),
 * gamma = trap*dt over n = batch*T*nheads f32 elements (trap already sigmoided, a_val <= 0). */
MRS_API int mrs_m3_compute_abg(void *stream, float *alpha, float *beta, float *gamma, const float *dt,
                               const float *a_val, const float *trap, int64_t n);

/* Chunked SSD forward: one call for the reference's adt product + m3_preprocess_chunks +
 * m3_dA_cumsum + m3_chunk_state_fwd + m3_state_passing_fwd + m3_chunk_scan_fwd +
 * m3_writeback_parallel_states (kernels/mamba3_chunked.cu:57-419, 1050-1242;
 * src/mamba3_siso/gpu/forward.rs:257-421).
 *   x,y [batch,T,d_inner] dtype; K,Q [batch,T,nheads,d_state] dtype (after bias+RoPE);
 *   dt, trap (sigmoided), a_val [batch,T,nheads] f32; D [nheads] f32.
 * flags = 0 is the reference's stateless window: the entering ssm/k/v state is ignored
 * (chunk 0 starts from zero, kernels/mamba3_chunked.cu:219-223) and the final state is
 * written back.  MRS_M3_CARRY_STATE continues from the entering state instead (prefill
 * after an earlier window, handing over to mrs_m3_step); the reference has no such mode.
 * chunk_size must be 64; headdim and d_state multiples of 16 with headdim <= 64, d_state <= 64
 * for the matrix-core path -- other shapes are refused (use mrs_m3_seq_fwd).  x, y, K, Q, ssm_state and k_state
 * 16-byte aligned (MRS_E_ALIGN otherwise): tiles are moved as 16-byte row pieces. */
enum { MRS_M3_CARRY_STATE = 1u << 0 };
MRS_API size_t mrs_m3_ssd_workspace_bytes(int batch, int T, int nheads, int headdim, int d_state, int chunk_size);
MRS_API int mrs_m3_ssd_fwd(void *stream, int dtype, float *ssm_state, float *k_state, float *v_state, void *y,
                           const void *x, const void *K, const void *Q, const float *dt, const float *trap,
                           const float *a_val, const float *D, void *workspace, size_t workspace_bytes,
                           unsigned flags, int batch, int T, int nheads, int headdim, int d_state,
                           int chunk_size);

/* ---- Mamba-1 backbone engine ----------------------------------------------------
 * The host surface of GpuMambaBackbone (src/mamba_ssm/gpu/inference.rs:1515-1855): the engine
 * owns device copies of the weights (projection matrices in `dtype`, the rest f32), the
 * persistent per-layer conv/SSM state and all scratch; nothing is allocated per step.
 * Host I/O is always f32.  Batch is fixed at creation.  An engine is not thread-safe
 * (the reference's is !Sync too, context.rs:16-56); it runs on its own non-blocking stream. */
typedef struct mrs_backbone mrs_backbone;

typedef struct {            /* MambaConfig, src/config.rs:57-84 */
    int d_model, d_state, d_conv, expand, n_layers;
    int scan_mode;          /* mrs_scan_mode */
    float rms_norm_eps;
} mrs_m1_config;

typedef struct {            /* MambaLayerWeights, src/weights.rs:7-42: host f32, row-major [n_in, n_out] */
    const float *norm_weight;   /* [d_model] */
    const float *in_proj_w;     /* [d_model, 2*d_inner] */
    const float *conv1d_weight; /* [d_inner, d_conv] */
    const float *conv1d_bias;   /* [d_inner] */
    const float *x_proj_w;      /* [d_inner, dt_rank + 2*d_state] */
    const float *dt_proj_w;     /* [dt_rank, d_inner] */
    const float *dt_proj_b;     /* [d_inner] */
    const float *a_log;         /* [d_inner, d_state]; a_neg = -exp(a_log) is derived at load */
    const float *d_param;       /* [d_inner] */
    const float *out_proj_w;    /* [d_inner, d_model] */
} mrs_m1_layer_weights;

typedef struct {            /* MambaWeights, src/weights.rs:51-64 */
    const float *input_proj_w;  /* [input_dim, d_model], or NULL for the identity (LM) case */
    const float *input_proj_b;  /* [d_model] or NULL (zeros) */
    const mrs_m1_layer_weights *layers; /* n_layers entries */
    const float *norm_f_weight; /* [d_model] */
} mrs_m1_weights;

/* ---- decode projections --------------------------------------------------------------------
 * The reference sends the decode chain's projections to cuBLAS (gemm_ex call sites
 * src/mamba_ssm/gpu/blas.rs:78-96, 721-737; tied head :709-740).  At batch <= 128 this library runs them
 * on its own matrix-core kernel over a TRANSPOSED weight.
 *   mrs_gemm_skinny: C[M,N] (row stride ldc; dtype, or f32 when out_f32) = A[M,K] (row stride lda) . Wt[N,K]^T
 *     dtype f16/bf16: 1 <= M <= 128, K % 32 == 0, lda % 8 == 0; f32: 1 <= M <= 4, K % 128 == 0, lda % 4 == 0; A and Wt
 *     16-byte aligned; f32 accumulate.
 *   mrs_transpose:   Wt[N,K] = W[K,N]^T (any dtype; builds the operand above from the reference's [K,N] layout). */
MRS_API int mrs_gemm_skinny(void *stream, int dtype, void *C, int out_f32, int64_t ldc, const void *A, int64_t lda,
                            const void *Wt, int M, int N, int K);
MRS_API int mrs_transpose(void *stream, int dtype, void *Wt, const void *W, int K, int N);
/* The same product from a TILED weight (what the decode chain reads from two or three rows up; wide models: in_proj of the 2.8b shape
 * is 52 MB): the 16 columns x 32 k of one matrix-core operand are 1 KB of consecutive memory, so the product is one
 * contiguous stream per wave (call sites src/mamba_ssm/gpu/blas.rs:1138-1163).
 *   mrs_tiled_weight_bytes: bytes of the tiled copy (columns padded to a multiple of 16); 0 for an unsupported dtype / K
 *   mrs_tile_weight:        Wp = tiled copy of the transposed weight Wt[N,K] (f16/bf16, K % 32 == 0, 16-byte aligned)
 *   mrs_gemm_tiled:         C[M,N] = A[M,K] . W; K % 32 == 0, lda % 8 == 0, A and Wp 16-byte aligned; 1 <= M <= 64 for a
 *                           weight of 16 MB or more (column-tile kernel), 1 <= M <= 128 below that (16 x 16 tiles) */
MRS_API size_t mrs_tiled_weight_bytes(int dtype, int N, int K);
MRS_API int mrs_tile_weight(void *stream, int dtype, void *Wp, const void *Wt, int N, int K);
MRS_API int mrs_gemm_tiled(void *stream, int dtype, void *C, int out_f32, int64_t ldc, const void *A, int64_t lda,
                           const void *Wp, int M, int N, int K);

/* GpuMambaBackbone::new_with_dtype(gpu_ordinal, &weights, cfg, input_dim, batch, dtype)  (inference.rs:1517-1575).
 * Validates the config with the reference's bounds (src/config.rs:108-170). */
MRS_API int mrs_backbone_create(mrs_backbone **out, int gpu_ordinal, const mrs_m1_weights *weights,
                                const mrs_m1_config *cfg, int input_dim, int batch, int dtype);
MRS_API void mrs_backbone_destroy(mrs_backbone *bb);
/* step(&[f32] input [batch*input_dim], &mut [f32] output [batch*d_model])  (inference.rs:1586): H2D, one
 * token through every layer, D2H, synchronises. */
MRS_API int mrs_backbone_step(mrs_backbone *bb, const float *input, float *output);
/* step_gpu_only (inference.rs:1670): input already in mrs_backbone_input_ptr(), output left in temporal_ptr(). */
MRS_API int mrs_backbone_step_gpu_only(mrs_backbone *bb);
/* reset (inference.rs:1599): zero conv and SSM state. */
MRS_API int mrs_backbone_reset(mrs_backbone *bb);
/* capture_graph (inference.rs:1608-1630): warm step, then capture the step body into a hipGraph that
 * step()/step_gpu_only() replay afterwards. State is preserved across the call. */
MRS_API int mrs_backbone_capture_graph(mrs_backbone *bb);
/* alloc_prefill_scratch / prefill_sequence[_mixed] (inference.rs:1752-1831; src/mamba_ssm/gpu/prefill.rs:676-1049):
 * input [batch, T, input_dim] f32 on the host; the whole sequence runs through the layers, the state ends
 * positioned after token T (so step continues), output_last (may be NULL) receives norm_f of the last position
 * [batch, d_model].  T >= 2.  The scratch follows T: kept while T repeats, released and re-made (device synchronise +
 * hipFree/hipMalloc) when a call brings another T -- the reference allocates it per call (src/module/gpu_lm.rs:543-551). */
MRS_API int mrs_backbone_alloc_prefill_scratch(mrs_backbone *bb, int T);
MRS_API int mrs_backbone_prefill_sequence(mrs_backbone *bb, const float *input, int T, float *output_last);
/* Same, input already on the device ([batch,T,input_dim] f32); does not synchronise. */
MRS_API int mrs_backbone_prefill_device(mrs_backbone *bb, const float *input_dev, int T);
/* Vendor-GEMM selection for the projections that go to the GEMM library: prefill, and decode steps of engines past the
 * own chain's row limit (no counterpart in the reference, which takes cuBLAS's default choice,
 * src/mamba_ssm/gpu/blas.rs:771-811).  With it on, the first call outside a stream capture that brings a projection
 * shape of 32 rows or more times every kernel the library offers for it (a few seconds per shape, once per engine) and
 * later calls use the fastest -- for decode that call is the eager step before mrs_backbone_capture_graph /
 * mrs_lm_capture_graph, so turn it on before capturing.  Results stay within the storage tolerance (another kernel sums
 * in another order).  Off by default; MRS_GEMM_TUNE=1 in the environment turns it on for every engine at creation. */
MRS_API int mrs_backbone_set_gemm_tuning(mrs_backbone *bb, int on);
/* temporal_ptr / input buffer / stream accessors (inference.rs:1717-1737) and state access for tests. */
MRS_API float *mrs_backbone_temporal_ptr(mrs_backbone *bb);
/* temporal_dtype (inference.rs:1720-1724): the dtype code of the buffer temporal_ptr returns.  This engine keeps that
 * buffer in f32 for every storage type, so the answer is MRS_F32; a caller that binds temporal_ptr must ask, because
 * the reference's mixed engine answers with its storage type. */
MRS_API int mrs_backbone_temporal_dtype(mrs_backbone *bb);
/* Which decode route the engine chose at creation (no counterpart in the reference; for tests and benchmarks that must
 * know what they measured): a whole step in one launch (small f32 models), the library's own fused kernel chain, or
 * the chain built on the vendor GEMM. */
#define MRS_DECODE_LIBRARY_CHAIN 0
#define MRS_DECODE_OWN_CHAIN 1
#define MRS_DECODE_ONE_LAUNCH 2
MRS_API int mrs_backbone_decode_route(mrs_backbone *bb);
/* download_temporal (inference.rs:1727-1737): the last step's / prefill's final-norm rows [batch, d_model] to the host; synchronises. */
MRS_API int mrs_backbone_download_temporal(mrs_backbone *bb, float *out);
MRS_API float *mrs_backbone_input_ptr(mrs_backbone *bb);
MRS_API float *mrs_backbone_prefill_input_ptr(mrs_backbone *bb);
MRS_API void *mrs_backbone_stream(mrs_backbone *bb);
MRS_API int mrs_backbone_sync(mrs_backbone *bb);
MRS_API int mrs_backbone_state_ptrs(mrs_backbone *bb, int layer, float **conv_state, float **ssm_state);
MRS_API int mrs_backbone_download_state(mrs_backbone *bb, int layer, float *conv_state, float *ssm_state);

/* ---- greedy LM loop on top of a backbone ------------------------------------------
 * The decode loop of GpuMambaLM::generate_streaming (src/module/gpu_lm.rs:334-377) with tied
 * embedding / lm_head (gpu_lm.rs:560-679), temperature 0: next token = last index of the maximum
 * logit (src/module/sample.rs:250-257).  Unlike the reference the embedding gather and the argmax
 * run on the device, so a decode step needs no host round trip.
 *   embed: [vocab, d_model] f32 on the host (rows >= vocab of the 64-padded table are zero). */
typedef struct mrs_lm mrs_lm;
MRS_API int mrs_lm_create(mrs_lm **out, mrs_backbone *decode_engine, const float *embed, int vocab);
/* A head with weights of its own (tie_word_embeddings = false; src/hf/load.rs:119-141, gpu_lm.rs:182-250):
 * lm_head is [d_model, vocab] f32 on the host.  Call before mrs_lm_capture_graph. */
MRS_API int mrs_lm_set_untied_head(mrs_lm *lm, const float *lm_head);
MRS_API void mrs_lm_destroy(mrs_lm *lm);
MRS_API int mrs_lm_set_tokens(mrs_lm *lm, const int *tokens);      /* [batch] current tokens */
MRS_API int mrs_lm_get_tokens(mrs_lm *lm, int *tokens);            /* synchronises */
MRS_API int mrs_lm_decode_step(mrs_lm *lm);                        /* tokens <- greedy next tokens */
MRS_API int mrs_lm_capture_graph(mrs_lm *lm);                      /* capture one decode step */
MRS_API int mrs_lm_last_logits(mrs_lm *lm, float *logits);         /* [batch, vocab] f32, synchronises */
/* tokens [prefill_engine.batch, T] -> embeddings -> prefill on `prefill_engine` (which may be the decode
 * engine itself, or null for it: then the head + argmax run and the next tokens are left in the token buffer). */
MRS_API int mrs_lm_prefill(mrs_lm *lm, mrs_backbone *prefill_engine, const int *tokens, int T);

/* ---- sampling and batched generation ------------------------------------------------------
 * sample_token (src/module/sample.rs:243-265): repetition penalty -> temperature -> top-k -> softmax -> top-p ->
 * min-p -> weighted draw, with the switches of SampleParams (sample.rs:20-46): temperature <= 0 is greedy (last
 * index of the maximum, no draw), top_k 0 / top_p outside (0,1) / min_p <= 0 / penalty 1, <= 0 or NaN are off.
 * The reference samples on the host from downloaded logits; here one launch samples every row on the device. */
typedef struct { float temperature; int top_k; float top_p; float min_p; float repetition_penalty; } mrs_sampler;

/* Xoshiro256PlusPlus::new (sample.rs:54-66): the four state words for a seed.  Host function. */
MRS_API void mrs_xoshiro_seed(unsigned long long seed, unsigned long long state[4]);

/* All pointers are device memory.  tokens [rows] <- sampled ids; logits [rows, ld] f32 (read only); work [rows, ld]
 * f32 scratch for the penalised rows (may be null when seen_counts is); samplers [rows]; seen_counts [rows, vocab] occurrences of each token in the row's seen list, or null
 * (no penalty); rng_state [rows, 4], advanced by one draw per sampled row; active [rows] or null: rows with 0 are
 * skipped (token, generator untouched). */
MRS_API int mrs_sample_tokens(void *stream, int *tokens, const float *logits, float *work, int64_t ld, int rows, int vocab,
                              const mrs_sampler *samplers, const unsigned *seen_counts, unsigned long long *rng_state,
                              const int *active);

/* SampleParams (sample.rs:20-46) of one slot; eos_token_ids may be null when n_eos is 0 (at most 16 ids). */
typedef struct {
    mrs_sampler sampler;
    int max_tokens;
    const int *eos_token_ids;
    int n_eos;
    unsigned long long seed;
} mrs_sample_params;

/* GpuMambaLM::generate_batch (src/module/gpu_lm.rs:389-516): one prompt per batch slot, of any length (an empty
 * prompt leaves its slot finished); prompts are consumed a token per step, slots whose prompt is done sample from
 * their own generator and stop at an EOS id or at max_tokens.  The whole loop -- gather, step, head, sampling and
 * the per-slot bookkeeping -- stays on the device; the host only polls how many slots are still running.
 *   prompts: all prompts back to back; prompt_lens [batch]; params [batch];
 *   out_tokens [batch, out_stride] and out_lens [batch] receive the generated ids (prompt excluded);
 *   out_stride >= every max_tokens.
 * seen_includes_prompt = 0: the penalty sees the generated tokens only (generate_batch, gpu_lm.rs:470-487);
 * 1: prompt and generated tokens (generate_streaming, gpu_lm.rs:364-375), and a batch-1 engine takes prompts of 256
 * tokens or more through prefill (gpu_lm.rs:349).  Resets the engine state, allocates its buffers on first use (and when
 * a call needs larger ones) and synchronises the engine's stream before it returns. */
MRS_API int mrs_lm_generate_batch(mrs_lm *lm, const int *prompts, const int *prompt_lens, const mrs_sample_params *params,
                                  int seen_includes_prompt, int *out_tokens, int out_stride, int *out_lens);

/* GpuMambaLM::generate_streaming (src/module/gpu_lm.rs:334-377), batch-1 engines: the loop of mrs_lm_generate_batch with
 * the penalty history over prompt + generated tokens and the prompt through the prefill path from 256 tokens on; every
 * new token is handed to `cb` as soon as it exists (one host round trip per step).  A nonzero return from `cb` ends the
 * generation early (the reference's callback cannot; returning 0 always reproduces it). */
typedef int (*mrs_token_callback)(int token, void *user);
MRS_API int mrs_lm_generate_streaming(mrs_lm *lm, const int *prompt, int prompt_len, const mrs_sample_params *params,
                                      mrs_token_callback cb, void *user);

/* ---- Mamba-3 SISO backbone engine (decode step) -------------------------------------------------
 * GpuMamba3Backbone (src/mamba3_siso/gpu/inference.rs:1487-1671): weights, per-layer state
 * (ssm [batch,nh,hd,ds], k [batch,nh,ds], v [batch,nh,hd], angle [batch,nh,n_rope], all f32) and scratch owned by
 * the engine; host I/O is f32.  One step per call for every batch row; the ten-phase layer of
 * step_layer_kernels (inference.rs:506-1000) is three kernels here.  Matrices are row-major [n_in, n_out]. */
typedef struct mrs_m3_backbone mrs_m3_backbone;

typedef struct {            /* Mamba3Config, src/mamba3_siso/config.rs:7-58 */
    int d_model, d_state, expand, headdim, ngroups, n_layers;
    int n_rope_angles;      /* num_rope_angles() = floor(d_state * rope_fraction) / 2 */
    float a_floor;          /* A <= -a_floor */
    int is_outproj_norm;    /* RMSNormGated before out_proj */
    float rms_norm_eps;     /* 1e-5 in the reference (ops/fast_math.rs:17) */
} mrs_m3_config;

typedef struct {            /* Mamba3LayerWeights, src/mamba3_siso/weights.rs:14-48 */
    const float *norm_weight;       /* [d_model] */
    const float *in_proj_w;         /* [d_model, in_proj_out_dim]: z | x | B | C | dd_dt | dd_A | trap | angles */
    const float *dt_bias;           /* [nheads] */
    const float *b_norm_weight;     /* [d_state] */
    const float *c_norm_weight;     /* [d_state] */
    const float *b_bias;            /* [nheads, d_state] */
    const float *c_bias;            /* [nheads, d_state] */
    const float *d_param;           /* [nheads] */
    const float *norm_gate_weight;  /* [d_inner] */
    const float *out_proj_w;        /* [d_inner, d_model] */
} mrs_m3_layer_weights;

typedef struct {            /* Mamba3Weights */
    const float *input_proj_w;  /* [input_dim, d_model], or NULL for the identity */
    const float *input_proj_b;  /* [d_model] or NULL (zeros) */
    const mrs_m3_layer_weights *layers;
    const float *norm_f_weight; /* [d_model] */
} mrs_m3_weights;

/* d_state = 4 x a power of two <= 256 and headdim * d_state / 4 a multiple of 64, <= 1024 (the reference stops at headdim 32). */
MRS_API int mrs_m3_backbone_create(mrs_m3_backbone **out, int gpu_ordinal, const mrs_m3_weights *weights,
                                   const mrs_m3_config *cfg, int input_dim, int batch, int dtype);
MRS_API void mrs_m3_backbone_destroy(mrs_m3_backbone *bb);
/* step(&mut self, input: &[f32], output: &mut [f32]): input [batch, input_dim] -> norm_f output [batch, d_model] */
MRS_API int mrs_m3_backbone_step(mrs_m3_backbone *bb, const float *input, float *output);
MRS_API int mrs_m3_backbone_step_gpu_only(mrs_m3_backbone *bb);   /* input already in input_ptr(), output left in temporal_ptr() */
MRS_API int mrs_m3_backbone_reset(mrs_m3_backbone *bb);
MRS_API int mrs_m3_backbone_capture_graph(mrs_m3_backbone *bb);
MRS_API float *mrs_m3_backbone_temporal_ptr(mrs_m3_backbone *bb);
/* temporal_dtype (src/mamba3_siso/gpu/inference.rs:1561-1563) and the decode route, as for the Mamba-1 engine */
MRS_API int mrs_m3_backbone_temporal_dtype(mrs_m3_backbone *bb);
MRS_API int mrs_m3_backbone_decode_route(mrs_m3_backbone *bb);
MRS_API float *mrs_m3_backbone_input_ptr(mrs_m3_backbone *bb);
MRS_API void *mrs_m3_backbone_stream(mrs_m3_backbone *bb);
MRS_API int mrs_m3_backbone_sync(mrs_m3_backbone *bb);
MRS_API int mrs_m3_backbone_download_state(mrs_m3_backbone *bb, int layer, float *ssm, float *k, float *v, float *angle);
/* Prefill: whole sequences [batch, T, input_dim] through the chunked SSD route (in_proj GEMM, angle prefix sums, the
 * split/bcnorm/bias/rope glue of kernels/mamba3_ops.cu in one kernel, mrs_m3_ssd_fwd with carried state, gate, out_proj),
 * continuing from the engine's state and leaving it positioned for step().  The reference's GPU forward of a layer over T
 * is gpu_forward_mamba3_layer (src/mamba3_siso/gpu/forward.rs:27); its CPU prefill mamba3_siso/cpu/prefill.rs:151-572.
 * The scratch follows T: allocated on first use or by alloc_prefill_scratch, re-made when a call brings another T. */
MRS_API int mrs_m3_backbone_alloc_prefill_scratch(mrs_m3_backbone *bb, int T);
MRS_API int mrs_m3_backbone_prefill_sequence(mrs_m3_backbone *bb, const float *input, int T, float *out_last);
MRS_API int mrs_m3_backbone_prefill_device(mrs_m3_backbone *bb, int T);
/* As mrs_backbone_set_gemm_tuning, for the Mamba-3 engine's in_proj / out_proj. */
MRS_API int mrs_m3_backbone_set_gemm_tuning(mrs_m3_backbone *bb, int on);
MRS_API float *mrs_m3_backbone_prefill_input_ptr(mrs_m3_backbone *bb);

/* GpuMamba3LM (src/module/gpu_lm3.rs:54-400): the LM loop over a Mamba-3 backbone (identity input_proj).  The handle is
 * an mrs_lm: every mrs_lm_* entry point above works on it (mrs_lm_prefill with a null prefill engine); the engine is
 * not owned.  embed: [vocab, d_model] f32 on the host. */
MRS_API int mrs_lm3_create(mrs_lm **out, mrs_m3_backbone *decode_engine, const float *embed, int vocab);

#ifdef __cplusplus
}
#endif
#endif /* MAMBA_HIP_H */
