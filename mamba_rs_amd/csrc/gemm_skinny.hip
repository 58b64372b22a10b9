// Skinny GEMM for the decode chain: C[M,N] = A[M,K] . Wt[N,K]^T with M <= 128 rows (the batch),
// 16-bit operands, f32 accumulate on the matrix cores.
//
// The reference sends every decode projection to the vendor GEMM (cuBLAS call sites
// src/mamba_ssm/gpu/blas.rs:78-96, 721-737).  At M <= 64 those calls are latency-bound: the work is a
// single pass over the weights (4.7 MB for in_proj at d_model 768), and what matters is that all of it is
// in flight at once and that the kernel ends as soon as the last byte has arrived.  Here:
//   * the weight is kept transposed, Wt[N][K], so that both MFMA operands are 16-byte row reads:
//     v_mfma_f32_16x16x32 takes A[m = l%16][k = 8(l/16)..+7] and B[k = 8(l/16)..+7][n = l%16], i.e. 8
//     consecutive k of activation row m and of weight row n (the k order inside the instruction is the
//     same for both operands, which is all a dot product needs);
//   * a workgroup owns a 16x16 output tile; its 8 waves split K (interleaved 32-wide steps), so a
//     K = 768 product is 3 steps per wave with every load independent; the partial tiles meet in LDS;
//   * the epilogue is fused: plain store (16-bit or f32), or in_proj's -- the x half of the row goes
//     straight through the depthwise conv step + SiLU (conv1d_step_forward_silu, kernels/conv1d.cu:85-115)
//     and only u and the gate half are written.
#include "common.hpp"
#include "mfma_tiles.hpp"
#include <stdlib.h>
#include <algorithm>

namespace mrs {

constexpr int kGemmWaves = 8;
constexpr int kMaxConvTaps = 8;

// 8 products of a 16-byte pair of operand chunks, f32 accumulate (v_dot2_f32_bf16 / v_dot2_f32_f16)
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
template <typename T> struct Dot2;
template <> struct Dot2<bf16_t> {
    __device__ static __forceinline__ float f(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf, a), __builtin_bit_cast(v2bf, b), c, false);
    }
};
template <> struct Dot2<f16_t> {
    __device__ static __forceinline__ float f(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2h, a), __builtin_bit_cast(v2h, b), c, false);
    }
};
// the products of one 16-byte piece of each operand: 8 elements of a 16-bit type (four v_dot2), 4 of f32
template <typename T> __device__ __forceinline__ float dot8(uint4 a, uint4 b, float c) {
    if constexpr (sizeof(T) == 4) {
        c = fmaf(__uint_as_float(a.x), __uint_as_float(b.x), c); c = fmaf(__uint_as_float(a.y), __uint_as_float(b.y), c);
        c = fmaf(__uint_as_float(a.z), __uint_as_float(b.z), c);
        return fmaf(__uint_as_float(a.w), __uint_as_float(b.w), c);
    } else {
        c = Dot2<T>::f(a.x, b.x, c); c = Dot2<T>::f(a.y, b.y, c); c = Dot2<T>::f(a.z, b.z, c);
        return Dot2<T>::f(a.w, b.w, c);
    }
}

template <typename TO> __device__ __forceinline__ void store_out(TO *p, float v) { Store<TO>::st(p, v); }

// EPI 0: C[row, col] = sum (TO = T or float)
// EPI 3: EPI 1 for any number of conv taps up to kMaxConvTaps (EPI 1 itself: four taps, window and taps one 16-byte
//        vector each, a third of the registers).
// EPI 1: in_proj of a Mamba-1 layer: columns < di are conv inputs (conv state [M][di][dc] f32 shifted in
//        place, u[row, col] = silu(conv)), columns >= di (the gate) are stored to C.
// Grid: x = 16-column tile, y = 16-row tile.  A workgroup pulls 16 rows of A and 16 rows of Wt through
// its L1 (49 KB each at K = 1536); measured, the time of this kernel is set by the bytes ONE workgroup has
// to pull (wider or taller tiles per workgroup were slower: 6.4 -> 7.5 us at 32 columns, 3.3 -> 6.4 us at
// 64 rows, K = 768), so tiles are kept minimal and the re-reads of Wt by the row tiles are left to L2.
constexpr int kStepsPerBatch = 6;  // k-steps whose loads are issued together (covers K <= 1536 in one round trip)

// PRO 1 (RMSNorm folded around the product): A holds round_T(residual[row,k] * norm_w[k]) -- the row scale
// 1/rms[row] commutes with the product, so it is applied to the f32 sums in the epilogue:
//   rmsnorm(x) . W = (1/rms) * ((x * w) . W)
// (rmsnorm_forward_f32in, kernels/norms.cu:21-171, with its guard rms = 1 when not finite or < 1e-20).
// rms comes from the row's partial sums of squares, which the out_proj epilogue before it (or
// prenorm_rows_kernel for the first layer) left behind together with A.  Against the reference's order the
// rounding to the storage type happens before the row scale instead of after it: same relative error.
//
// LPR != 0 (M <= 4, one row tile): no matrix cores.  At one to four rows the product is a pass over the weight and
// nothing else, so the layout follows the memory system: LPR lanes (64 or 32) walk one weight row in consecutive
// 16-byte pieces -- whole kilobytes of one row per load instruction instead of 64-byte pieces of 16 rows -- each wave
// owns two of the workgroup's 16 columns, all of its loads are in flight at once (in groups of JB per column), and
// the products are v_dot2 with f32 accumulate.  The epilogues are the same code.  MR = rows computed (1, 2 or 4; at 8 rows the route was slower than the matrix-core tiles: 642 vs 435 us per 130m-shape step).
template <typename T, typename TO, int EPI, int PRO, int LPR = 0, int MR = 1>
__global__ __launch_bounds__(kGemmWaves * 64) __attribute__((amdgpu_waves_per_eu(6))) void skinny_gemm_kernel(
    TO *__restrict__ C, int64_t ldc, const T *__restrict__ A, int64_t lda, const T *__restrict__ Wt, int M, int N, int K,
    SkinnyEpi ep) {
    __shared__ v4f red[LPR ? 1 : kGemmWaves][kWave];
    __shared__ float gv[4][16];   // LPR != 0: the [row][column] sums of the workgroup
    const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16;
    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, lr = l & 15, lg = l >> 4;
    // k-steps of this workgroup: all of them, or slice blockIdx.z of gridDim.z (matrix-core route, plain store only)
    const int nk_all = K >> 5;
    const int k_lo = LPR == 0 ? (int)blockIdx.z * ep.kslice : 0;
    const int nk = LPR == 0 ? min(nk_all, k_lo + ep.kslice) : nk_all;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    // Rows past M / columns past N are clamped to the last valid one: their products land in
    // accumulator elements that are never stored.
    constexpr int EPV = 16 / (int)sizeof(T);   // elements per 16-byte piece
    // Matrix-core route: either operand may be stored tiled -- the 16 x 32 piece of one matrix instruction as 1 KB in lane
    // order (gemm_wide.hip: launch_tile_weight, tiled_a_index) -- so that a fragment load is one contiguous kilobyte
    // instead of sixteen 64-byte row pieces: eight cache lines for the L1 to look up instead of sixty-four, which is what
    // these short products are bound by (64 x 3072 x 768: 6.6 us row-major, 4.4 us tiled).
    const bool w_tiled = LPR == 0 && ep.w_tiled, a_tiled = LPR == 0 && ep.a_tiled;
    const T *wrow = w_tiled ? Wt + (int64_t)(n0 >> 4) * (K >> 5) * 512 + 8 * l : Wt + (int64_t)min(n0 + lr, N - 1) * K + 8 * lg;
    const T *arow = a_tiled ? A + (int64_t)(m0 >> 4) * 512 + 8 * l : A + (int64_t)min(m0 + lr, M - 1) * lda + 8 * lg;
    const int wks = w_tiled ? 512 : 32, aks = a_tiled ? 512 * ((M + 15) >> 4) : 32;   // elements from one k-step's piece to the next
    float inv = 1.0f;
    // The partial sums of a row are requested together, right behind the first operand requests, and added up at once in
    // the order a loop over them would add them (loads come back in the order they were issued, so this waits for nothing
    // the first products do not wait for as well).  Loaded one at a time inside such a loop they were a chain of
    // n_partials / 16 round trips to L2 ahead of the first operand request (ten at d_model 2560); requested ahead of the
    // operands and kept until after the product, three of the eight were spilled under this kernel's register limit, each
    // behind a wait of its own for its load.
    // Partial sums per lane requested together; any beyond are loaded late.  Matrix-core route: the 16 lanes of an
    // epilogue row share them, four each (narrow models: d_model up to 1024 without a late load; no registers to spare
    // for more under this kernel's limit).  Row-wise route (up to four rows): wave m sums row m, four per lane cover 256
    // partial sums, and the rows' scales meet the epilogue threads in LDS.
    constexpr int kScaleAhead = 4;
    constexpr int kScaleLanes = LPR == 0 ? 16 : 64;
    __shared__ float inv_rows[4];
    float ss_ahead;                           // set by row_scale_fold alone (an addition to a preset would be made at the loads)
    float psum[PRO == 1 ? kScaleAhead : 1];   // no presets, no branch around a load: see prefetch_epilogue
    const bool scale_thread = PRO == 1 && (LPR == 0 ? tid < 256 : w < MR);   // the same for a whole wave
    const int scale_row = m0 + (LPR == 0 ? (tid >> 4) : w), scale_lane = LPR == 0 ? (tid & 15) : l;
    auto row_scale_request = [&]() {
        if (scale_thread) {
            const float *pp = ep.partials + (int64_t)min(scale_row, M - 1) * ep.n_partials;
#pragma unroll
            for (int j = 0; j < kScaleAhead; j++) psum[j] = pp[min(scale_lane + kScaleLanes * j, ep.n_partials - 1)];
        }
    };
    auto row_scale_fold = [&]() {
        if (scale_thread) {
            float a = scale_lane < ep.n_partials ? psum[0] : 0.0f;
#pragma unroll
            for (int j = 1; j < kScaleAhead; j++) a += scale_lane + kScaleLanes * j < ep.n_partials ? psum[j] : 0.0f;
            ss_ahead = a;
        }
    };
    auto row_scale = [&]() {
        if (scale_thread) {
            const float *pp = ep.partials + (int64_t)min(scale_row, M - 1) * ep.n_partials;
            float ss = ss_ahead;
            if (ep.n_partials > kScaleLanes * kScaleAhead) {   // a wider row: the next eight per lane as one more round trip, then one at a time
                float late[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int p = scale_lane + kScaleLanes * (kScaleAhead + j);
                    late[j] = p < ep.n_partials ? pp[p] : 0.0f;
                }
#pragma unroll
                for (int j = 0; j < 8; j++) ss += late[j];
                for (int p = scale_lane + kScaleLanes * (kScaleAhead + 8); p < ep.n_partials; p += kScaleLanes) ss += pp[p];
            }
#pragma unroll
            for (int m = kScaleLanes / 2; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
            float rms = sqrtf(ss / (float)K + ep.eps);
            if (!isfinite(rms) || rms < 1e-20f) rms = 1.0f;
            inv = 1.0f / rms;
            if (LPR != 0 && l == 0) inv_rows[w] = inv;   // published by the barrier behind the products
        }
    };
    // Epilogue operands that do not depend on the product -- the conv window / taps / bias (mode 1), the
    // residual element and next norm weight (mode 2) -- can be requested before the operands stream.
    const int e_row = m0 + (tid >> 4), e_col = n0 + (tid & 15);
    const bool e_valid = tid < 256 && e_row < M && e_col < N;
    constexpr bool kConv = EPI == 1 || EPI == 3;
    constexpr int kTaps = EPI == 3 ? kMaxConvTaps : 4;
    // No presets and no branch that depends on the lane around a load: a value that is a load on one path and a constant
    // on another has to be copied into place once the load is back, and the compiler waits for the load right there --
    // each of these requests then cost a memory round trip of its own in front of the product.  Lanes whose element lies
    // outside the result load from a clamped (row, column) and never use what they get.
    float win[kTaps], cwv[kTaps], cbias, res_old, nw;
    auto prefetch_epilogue = [&]() {
        if (tid < 256) {   // the same for a whole wave
            const int r = min(e_row, M - 1), c = min(e_col, N - 1);
            if constexpr (kConv) {
                const int cc = min(c, ep.di - 1);
                const float *st = ep.conv_state + ((int64_t)r * ep.di + cc) * ep.dc;
                const float *cw = ep.conv_w + (int64_t)cc * ep.dc;
                if constexpr (EPI == 1) {   // four taps: window and taps are one aligned 16-byte vector each
                    const float4 s4 = *reinterpret_cast<const float4 *>(st), c4 = *reinterpret_cast<const float4 *>(cw);
                    win[0] = s4.y; win[1] = s4.z; win[2] = s4.w; win[3] = 0.0f;
                    cwv[0] = c4.x; cwv[1] = c4.y; cwv[2] = c4.z; cwv[3] = c4.w;
                } else {
#pragma unroll
                    for (int k = 0; k < kTaps; k++) {
                        win[k] = (k + 1 < ep.dc) ? st[k + 1] : 0.0f;
                        cwv[k] = (k < ep.dc) ? cw[k] : 0.0f;
                    }
                }
                cbias = ep.conv_b[cc];
            }
            if constexpr (EPI == 2) {
                const float *pr = ep.residual + (int64_t)r * N + c;
                res_old = *pr;
                nw = *(ep.next_norm_w ? ep.next_norm_w + c : pr);   // used only with a next norm weight
            }
        }
    };
    // every request first, then the first use of any of them (left to itself the scheduler puts the first partial sum's
    // addition in front of the epilogue's requests, which then start a memory round trip late)
    auto early_requests = [&]() {
        row_scale_request();
        prefetch_epilogue();
        __builtin_amdgcn_sched_barrier(0);
        row_scale_fold();
    };
    // Requested up front, but on the matrix-core route behind the first round of operand loads: with several row
    // tiles the conv windows are a megabyte-scale read that would otherwise queue ahead of the operands.
    if constexpr (LPR != 0) {
        constexpr int NC = LPR == 64 ? 2 : 1;           // columns a lane works on (with 32 lanes per row each half-wave has its own)
        constexpr int JB = LPR == 64 ? 2 : 4;             // pieces per column requested together
        const int ll = l & (LPR - 1), half = LPR == 64 ? 0 : (l >> 5);
        const int per = (K / EPV) / LPR;                 // 16-byte pieces of a row per lane
        const T *wp[NC];
#pragma unroll
        for (int t = 0; t < NC; t++) wp[t] = Wt + (int64_t)min(n0 + 2 * w + (LPR == 64 ? t : half), N - 1) * K + EPV * ll;
        float sum[NC][MR];
#pragma unroll
        for (int t = 0; t < NC; t++)
#pragma unroll
            for (int m = 0; m < MR; m++) sum[t][m] = 0.0f;
        if constexpr (MR == 1) {
            // one row: each lane reads its own pieces of it next to the weight pieces (the row is 1/2 of a wave's bytes)
            constexpr int J1 = 4;
            for (int jb = 0; jb < per; jb += J1) {
                uint4 wv[NC][J1], av[J1];
#pragma unroll
                for (int j = 0; j < J1; j++) {
                    if (jb + j < per) {
                        const int off = EPV * LPR * (jb + j);
#pragma unroll
                        for (int t = 0; t < NC; t++) wv[t][j] = *reinterpret_cast<const uint4 *>(wp[t] + off);
                        av[j] = *reinterpret_cast<const uint4 *>(A + EPV * ll + off);
                    }
                }
                // the row's partial sums and the epilogue's operands behind the first weight requests (ahead of them, the
                // conv sum the compiler starts from window, taps and bias alone waited for the cold conv windows before
                // any weight was asked for)
                if (jb == 0) { early_requests(); }
#pragma unroll
                for (int j = 0; j < J1; j++) {
                    if (jb + j < per) {
#pragma unroll
                        for (int t = 0; t < NC; t++) sum[t][0] = dot8<T>(av[j], wv[t][j], sum[t][0]);
                    }
                }
            }
        } else {
        // two to four rows go through LDS once per workgroup: read per wave from memory they would add M/2 times the
        // weight bytes to what the workgroup pulls through its L1, which is what bounds this kernel
        extern __shared__ uint4 a_lds[];                // [MR][K / EPV]
        const int kq = K / EPV;
        for (int i = tid; i < MR * kq; i += kGemmWaves * 64) {
            const int m = i / kq, q = i - m * kq;
            a_lds[i] = *reinterpret_cast<const uint4 *>(A + (int64_t)min(m, M - 1) * lda + EPV * q);
        }
        // the first round of weight loads is issued before the barrier that publishes the rows
        uint4 wv[NC][JB];
#pragma unroll
        for (int j = 0; j < JB; j++)
            if (j < per) {
#pragma unroll
                for (int t = 0; t < NC; t++) wv[t][j] = *reinterpret_cast<const uint4 *>(wp[t] + EPV * LPR * j);
            }
        early_requests();
        lds_barrier();   // the rows are in LDS; the weight loads above stay in flight
        for (int jb = 0; jb < per; jb += JB) {
            uint4 nx[NC][JB];
#pragma unroll
            for (int j = 0; j < JB; j++)
                if (jb + JB + j < per) {
#pragma unroll
                    for (int t = 0; t < NC; t++) nx[t][j] = *reinterpret_cast<const uint4 *>(wp[t] + EPV * LPR * (jb + JB + j));
                }
#pragma unroll
            for (int j = 0; j < JB; j++) {
                if (jb + j < per) {
#pragma unroll
                    for (int m = 0; m < MR; m++) {
                        const uint4 av = a_lds[m * kq + ll + LPR * (jb + j)];
#pragma unroll
                        for (int t = 0; t < NC; t++) sum[t][m] = dot8<T>(av, wv[t][j], sum[t][m]);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < JB; j++)
#pragma unroll
                for (int t = 0; t < NC; t++) wv[t][j] = nx[t][j];
        }
        }
        row_scale();
#pragma unroll
        for (int t = 0; t < NC; t++)
#pragma unroll
            for (int m = 0; m < MR; m++) {
                float v = sum[t][m];
#pragma unroll
                for (int x = LPR / 2; x >= 1; x >>= 1) v += __shfl_xor(v, x, kWave);
                if (ll == 0) gv[m][2 * w + (LPR == 64 ? t : half)] = v;
            }
        lds_barrier();
    } else if constexpr (sizeof(T) == 2) {
    // Two half-batches of fragments: the next one is requested as soon as the current one has been multiplied, so a
    // long K (wide models: 20 k-steps per wave at K = 5120) streams instead of draining after every round of loads.
    constexpr int kHalf = kStepsPerBatch / 2;
    uint4 bf[2][kHalf], af[2][kHalf];
    auto request = [&](int h, int base) {
#pragma unroll
        for (int s = 0; s < kHalf; s++) {
            const int ks = base + s * kGemmWaves;
            // steps past K multiply zeros (every fragment is defined on every path)
            bf[h][s] = ks < nk ? *reinterpret_cast<const uint4 *>(wrow + wks * ks) : make_uint4(0, 0, 0, 0);
            af[h][s] = ks < nk ? *reinterpret_cast<const uint4 *>(arow + aks * ks) : make_uint4(0, 0, 0, 0);
        }
    };
    constexpr int kStride = kGemmWaves * kHalf;   // k-steps one half-batch covers across the workgroup's waves
    request(0, k_lo + w);
    request(1, k_lo + w + kStride);
    early_requests();
    for (int base = k_lo + w; base < nk; base += 2 * kStride) {
#pragma unroll
        for (int s = 0; s < kHalf; s++) acc = Mma32<T>::mma(af[0][s], bf[0][s], acc);
        request(0, base + 2 * kStride);   // past K: zeros, so a half-batch is never multiplied twice
#pragma unroll
        for (int s = 0; s < kHalf; s++) acc = Mma32<T>::mma(af[1][s], bf[1][s], acc);
        request(1, base + 3 * kStride);
    }
    row_scale();
    // K-split reduction: every wave parks its tile in LDS; the thread that owns an element adds them in wave order
    red[w][l] = acc;
    lds_barrier();   // LDS exchanges only: the epilogue's prefetched operands stay in flight
    }
    // element e of the 16x16 tile: row ml = e / 16, column nl = e % 16 lives in lane 16 (ml / 4) + nl, register ml % 4
    float u_out = 0.0f;   // mode 1: this thread's u as stored (0 for gate columns / rows past M)
    if (tid < 256) {
        const int ml = tid >> 4, nl = tid & 15;
        const int lane = (ml >> 2) * 16 + nl, i = ml & 3;
        float s = 0.0f;
        if constexpr (LPR != 0) {
            s = ml < MR ? gv[ml & 3][nl] : 0.0f;
        } else {
#pragma unroll
            for (int ww = 0; ww < kGemmWaves; ww++) s += red[ww][lane][i];
        }
        if constexpr (LPR != 0 && PRO == 1) inv = inv_rows[ml < MR ? ml : 0];
        s *= inv;
        const int row = m0 + ml, col = n0 + nl;
        const bool valid = row < M && col < N;
        if (EPI == 2) {
            // out_proj: residual += out (rounded to the storage type as the stored projection would be); the
            // row's sum of squares over these 16 columns and the pre-scaled operand for the next layer's in_proj
            float sq = 0.0f;
            if (valid) {
                const T orr = (T)s;
                const float rn = res_old + Store<T>::ld(&orr);
                ep.residual[(int64_t)row * N + col] = rn;
                sq = rn * rn;
                if (ep.next_norm_w)
                    Store<T>::st(reinterpret_cast<T *>(ep.prenorm) + (ep.prenorm_mt ? tiled_a_index(row, col, ep.prenorm_mt) : (int64_t)row * N + col), rn * nw);
            }
#pragma unroll
            for (int m = 8; m >= 1; m >>= 1) sq += __shfl_xor(sq, m, kWave);
            if (nl == 0 && row < M) ep.partials[(int64_t)row * ep.n_partials + blockIdx.x] = sq;
        } else if (!valid) {
        } else if (kConv && col < ep.di) {
            // conv step on the value as in_proj would have stored it (rounded to the storage type)
            const T xr = (T)s;
            const float xnew = Store<T>::ld(&xr);
            float *st = ep.conv_state + ((int64_t)row * ep.di + col) * ep.dc;
            float o = cbias;
            if constexpr (EPI == 1) {
                o = fmaf(win[0], cwv[0], o); o = fmaf(win[1], cwv[1], o); o = fmaf(win[2], cwv[2], o); o = fmaf(xnew, cwv[3], o);
                *reinterpret_cast<float4 *>(st) = make_float4(win[0], win[1], win[2], xnew);
            } else {
#pragma unroll
                for (int k = 0; k < kTaps; k++)
                    if (k < ep.dc) {
                        const float wk = (k + 1 < ep.dc) ? win[k] : xnew;
                        o = fmaf(wk, cwv[k], o);
                        st[k] = wk;
                    }
            }
            const T ur = (T)silu(o);
            reinterpret_cast<T *>(ep.u)[(int64_t)row * ep.di + col] = ur;
            if (ep.u_tiled) reinterpret_cast<T *>(ep.u_tiled)[tiled_a_index(row, col, ep.u_tiled_mt)] = ur;   // x_proj's operand
            u_out = Store<T>::ld(&ur);
        } else if (EPI == 0 && LPR == 0 && gridDim.z > 1) {
            ep.xpart[((int64_t)blockIdx.z * M + row) * N + col] = s;   // this slice's share, summed by the reader
        } else {
            store_out<TO>(C + (int64_t)row * ldc + col, s);
        }
    }
    if constexpr (kConv) {
        if (ep.xw != nullptr && n0 < ep.di) {   // the same for the whole workgroup
            // this tile's share of the x_proj rows: u[row, 16 columns] . W[16 columns, xd], f32, into [tile][row][xd]
            __shared__ float ush[16][16];
            if (tid < 256) ush[tid >> 4][tid & 15] = u_out;
            lds_barrier();
            const int xd = ep.xd, rows_here = min(16, M - m0);
            const T *xw = reinterpret_cast<const T *>(ep.xw);
            float *dst = ep.xpart + ((int64_t)blockIdx.x * M + m0) * xd;
            for (int o = tid; o < rows_here * xd; o += kGemmWaves * 64) {
                const int m = o / xd, j = o - m * xd;
                float a = 0.0f;
#pragma unroll
                for (int c = 0; c < 16; c++) a = fmaf(ush[m][c], Store<T>::ld(xw + (int64_t)min(n0 + c, ep.di - 1) * xd + j), a);
                dst[o] = a;
            }
        }
    }
}

// First layer's share of the folded norm: partials[row][0] = sum_k x[row][k]^2 (other slots zero) and
// prenorm[row][k] = round_T(x[row][k] * w[k]), for a residual stream no out_proj epilogue has produced yet;
// copy_to (may be null) also receives x, so the step's input buffer can feed the residual stream directly.
template <typename T>
__global__ __launch_bounds__(256) void prenorm_rows_kernel(float *__restrict__ partials, int n_partials, T *__restrict__ prenorm,
                                                           const float *__restrict__ x, float *__restrict__ copy_to,
                                                           const float *__restrict__ w, int K, int a_mt) {
    __shared__ float part[4];
    const int64_t row = blockIdx.x;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < K; i += 256) {
        const float v = x[row * K + i];
        ss = fmaf(v, v, ss);
        if (copy_to) copy_to[row * K + i] = v;   // the residual stream, when x is the step's input buffer
        Store<T>::st(prenorm + (a_mt ? tiled_a_index((int)row, i, a_mt) : row * K + i), v * w[i]);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    for (int p = threadIdx.x; p < n_partials; p += 256) partials[row * n_partials + p] = p == 0 ? part[0] + part[1] + part[2] + part[3] : 0.0f;
}


// Prefill dt_proj with its bias and softplus fused: delta[r, d] = softplus(round_T(sum_k dt_in[r, k] dt_w[k, d]) + bias[d]).
// The reference runs a GEMM with K = dt_rank, then bias add and softplus_forward (src/mamba_ssm/gpu/prefill.rs:846-905,
// kernels/activations.cu:32-52).  K is tiny (48 at d_model 768), so the op is one write of delta (50 MB per layer at the
// 130m prefill shape) and the softplus arithmetic.  dt_in rows have stride xs (they are the head of the x_proj row); wt is
// [d_inner][dt_rank].  KS = 32-wide k-steps (dt_rank <= 32 KS, K zero-padded), CT = 16-column tiles per workgroup.
//
// The product is formed TRANSPOSED: the weight is the matrix instruction's first operand and the 16 rows of a wave its
// second, so a lane's four results of one instruction are four COLUMNS of one row.  Operand row m of column tile ct stands
// for column 64 (ct / 4) + 16 (m / 4) + 4 (ct % 4) + m % 4 of the workgroup's block: after the four tiles of a 64-column
// sub-block a lane holds 16 consecutive columns of its row, which leave as two 16-byte stores -- the four lane groups of a
// row fill a 128-byte line, with no transpose through LDS (which the row-major product needed: 16 two-byte LDS writes per
// lane and tile).  A workgroup owns 16 CT columns and walks row tiles blockIdx.y, blockIdx.y + gridDim.y, ...: weight
// operands and bias are loaded once, the next tile's rows are requested while the current tile is in its epilogue.
// WLDS: the weight operands live in LDS, in operand order (one conflict-free kilobyte per matrix instruction), instead of
// registers: from dt_rank 97 up (KS >= 4: the 2.8b shape has dt_rank 160) 16 registers per k-step and sub-block for them
// would leave two waves per SIMD.  There the workgroup owns 128 columns: every column block re-reads the dt_in rows
// (6.3 MB at 4 x 4096 rows) through L2, 40 blocks instead of 80.
// What the kernel costs is its arithmetic: per result ten plain and two transcendental instructions (rounding the
// projection to the storage type and back, bias, softplus, packing).  Measured per layer, 130m prefill shape (50 MB of
// delta) / 2.8b shape (168 MB): the row-major product with its LDS transpose and a twelve-slot softplus 21.4 / 94 us; this
// kernel with the same softplus 21.1 / 93; with softplus20_16 as it is now 20.3 / 84.8; with the row tiles dealt evenly
// among the workgroups (launch_dt_proj_softplus) 18.7 / 77.2.
template <typename T, int KS, int CT, bool WLDS>
__global__ __launch_bounds__(256) void dt_proj_softplus_kernel(T *__restrict__ delta, const T *__restrict__ dt_in, int64_t xs,
                                                               const T *__restrict__ wt, const float *__restrict__ bias, int64_t rows,
                                                               int di, int dr) {
    static_assert(CT % 4 == 0, "whole 64-column sub-blocks");
    constexpr int SB = CT / 4;
    __shared__ uint4 wl[WLDS ? CT * KS * 64 : 1];   // [column tile][k-step][lane]
    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, lr = l & 15, lg = l >> 4;
    const int n0 = blockIdx.x * (16 * CT);
    const int64_t n_tiles = (rows + 63) / 64;
    // the weight piece that lane `lane` brings to the instruction of (column tile ct, k-step ks)
    auto weight_piece = [&](int ct, int ks, int lane) {
        const int m = lane & 15, k = 32 * ks + 8 * (lane >> 4);   // dt_rank % 8 == 0: a lane's 8 values are all inside or all outside
        const int col = min(n0 + 64 * (ct >> 2) + 16 * (m >> 2) + 4 * (ct & 3) + (m & 3), di - 1);
        return k < dr ? *reinterpret_cast<const uint4 *>(wt + (int64_t)col * dr + k) : make_uint4(0, 0, 0, 0);
    };
    uint4 wf[WLDS ? 1 : KS][WLDS ? 1 : CT];
    if constexpr (WLDS) {
        for (int i = tid; i < CT * KS * 64; i += 256) wl[i] = weight_piece((i >> 6) / KS, (i >> 6) % KS, i & 63);
        __syncthreads();
    } else {
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++) wf[ks][ct] = weight_piece(ct, ks, l);
    }
    float bv[SB][16];   // bias of this lane's 16 consecutive columns per sub-block
#pragma unroll
    for (int sb = 0; sb < SB; sb++)
#pragma unroll
        for (int j = 0; j < 16; j++) bv[sb][j] = bias[min(n0 + 64 * sb + 16 * lg + j, di - 1)];
    // Rows of tile rt.  Every load and every store is issued on every path -- past the last tile the last one again, past
    // the last row the last row again (its lanes then hold, and store, the same values), past dt_rank the row's own next
    // values (B and C of the x_proj row), which meet zero weights.  Behind conditions the compiler waited for the NEXT
    // tile's rows in front of the current tile's matrix instructions, and for the stores of a tile before the next.
    auto load_rows = [&](int64_t rt, uint4 (&rf)[KS]) {
        const int64_t row = min(min(rt, n_tiles - 1) * 64 + 16 * w + lr, rows - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) rf[ks] = *reinterpret_cast<const uint4 *>(dt_in + row * xs + min(32 * ks + 8 * lg, (int)xs - 8));
    };
    uint4 rf[KS];
    int64_t rt = blockIdx.y;
    load_rows(rt, rf);
    for (; rt < n_tiles; rt += gridDim.y) {
        const int64_t row = min(rt * 64 + 16 * w + lr, rows - 1);
        // (the weight operands are read from LDS where they are used: hoisted out of this loop they are 128 registers and more)
        if constexpr (WLDS) asm volatile("" ::: "memory");
        v4f acc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ct++) {
            acc[ct] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                uint4 wv;
                if constexpr (WLDS) wv = wl[(ct * KS + ks) * 64 + l];
                else wv = wf[ks][ct];
                acc[ct] = Mma32<T>::mma(wv, rf[ks], acc[ct]);
            }
        }
        load_rows(rt + gridDim.y, rf);   // the next tile's rows travel during this tile's epilogue
#pragma unroll
        for (int sb = 0; sb < SB; sb++) {
            alignas(16) T out[16];
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const T raw = (T)acc[4 * sb + (j >> 2)][j & 3];   // the projection as the reference stores it, before bias and softplus
                Store<T>::st(&out[j], softplus20_16(Store<T>::ld(&raw) + bv[sb][j]));
            }
            T *dst = delta + row * di + n0 + 64 * sb + 16 * lg;
            *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(&out[0]);
            *reinterpret_cast<uint4 *>(dst + 8) = *reinterpret_cast<const uint4 *>(&out[8]);
        }
    }
}

// Wt[n][k] = W[k][n]: 32x32 tiles through LDS so both sides are coalesced.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(T *__restrict__ Wt, const T *__restrict__ W, int K, int N) {
    __shared__ T tile[32][33];
    const int k0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int r = ty; r < 32; r += 8)
        if (k0 + r < K && n0 + tx < N) tile[r][tx] = W[(int64_t)(k0 + r) * N + n0 + tx];
    __syncthreads();
    for (int r = ty; r < 32; r += 8)
        if (n0 + r < N && k0 + tx < K) Wt[(int64_t)(n0 + r) * K + k0 + tx] = tile[tx][r];
}

static bool no_rowwise_route() {
    static const bool v = getenv("MRS_DECODE_NO_ROWWISE") != nullptr;
    return v;
}

template <typename T, typename TO>
static int launch_skinny_t(hipStream_t st, TO *C, int64_t ldc, const T *A, int64_t lda, const T *Wt, int M, int N, int K,
                           const SkinnyEpi &ep_in) {
    SkinnyEpi ep = ep_in;
    const dim3 block(kGemmWaves * 64);
    // one to four rows: the lanes-along-the-row route (64 lanes per weight row when a row is a multiple of 1 KB, else 32)
    constexpr int EPV = 16 / (int)sizeof(T);   // elements per 16-byte piece
    const bool no_rowwise = no_rowwise_route();
    int lpr = (M > 4 || no_rowwise || (int64_t)K * 4 * sizeof(T) > 48 * 1024) ? 0   // four rows must fit in LDS
                                                                               : (K % (64 * EPV) == 0 ? 64 : (K % (32 * EPV) == 0 ? 32 : 0));
    const int ksplit = (ep.mode == 0 && ep.ksplit > 1) ? ep.ksplit : 1;
    if (ksplit > 1) lpr = 0;   // a split K runs on the matrix-core route at any row count
    if (ep.w_tiled || ep.a_tiled) lpr = 0;   // tiled operands are matrix-core operands
    if (sizeof(T) == 4 && lpr == 0) return fail(MRS_E_SHAPE, "skinny gemm: f32 storage runs on the row-wise route only (M <= 4, K %% 128 == 0, no K split)");
    if (ksplit > 1 && (ep.row_scale || !ep.xpart || ksplit > (K >> 5)))
        return fail(MRS_E_SHAPE, "skinny gemm: K split needs the matrix-core route, a plain product, a share buffer and ksplit <= K / 32 (ksplit=%d)", ksplit);
    ep.kslice = ((K >> 5) + ksplit - 1) / ksplit;
    const dim3 grid((unsigned)((N + 15) / 16), (unsigned)((M + 15) / 16), (unsigned)(((K >> 5) + ep.kslice - 1) / ep.kslice));
#define MRS_SG(EPI_, PRO_)                                                                                                               \
    do {                                                                                                                                 \
        if (lpr == 64 && M == 1) hipLaunchKernelGGL((skinny_gemm_kernel<T, TO, EPI_, PRO_, 64, 1>), grid, block, 0, st, C, ldc, A, lda, Wt, M, N, K, ep); \
        else if (lpr == 64 && M == 2) hipLaunchKernelGGL((skinny_gemm_kernel<T, TO, EPI_, PRO_, 64, 2>), grid, block, (size_t)K * 2 * sizeof(T), st, C, ldc, A, lda, Wt, M, N, K, ep); \
        else if (lpr == 32 && M == 2) hipLaunchKernelGGL((skinny_gemm_kernel<T, TO, EPI_, PRO_, 32, 2>), grid, block, (size_t)K * 2 * sizeof(T), st, C, ldc, A, lda, Wt, M, N, K, ep); \
        else if (lpr == 64) hipLaunchKernelGGL((skinny_gemm_kernel<T, TO, EPI_, PRO_, 64, 4>), grid, block, (size_t)K * 4 * sizeof(T), st, C, ldc, A, lda, Wt, M, N, K, ep);     \
        else if (lpr == 32 && M == 1) hipLaunchKernelGGL((skinny_gemm_kernel<T, TO, EPI_, PRO_, 32, 1>), grid, block, 0, st, C, ldc, A, lda, Wt, M, N, K, ep); \
        else if (lpr == 32) hipLaunchKernelGGL((skinny_gemm_kernel<T, TO, EPI_, PRO_, 32, 4>), grid, block, (size_t)K * 4 * sizeof(T), st, C, ldc, A, lda, Wt, M, N, K, ep);     \
        else hipLaunchKernelGGL((skinny_gemm_kernel<T, TO, EPI_, PRO_>), grid, block, 0, st, C, ldc, A, lda, Wt, M, N, K, ep);           \
    } while (0)
    const bool pro = ep.row_scale != 0;
    if (ep.mode != 0 && sizeof(TO) != sizeof(T)) return fail(MRS_E_DTYPE, "skinny gemm: fused epilogues store the activation type");
    if constexpr (sizeof(TO) == sizeof(T)) {
        if (ep.mode == 1 && ep.dc == 4) { if (pro) MRS_SG(1, 1); else MRS_SG(1, 0); return check_launch("skinny_gemm_kernel"); }
        if (ep.mode == 1) { if (pro) MRS_SG(3, 1); else MRS_SG(3, 0); return check_launch("skinny_gemm_kernel"); }
        if (ep.mode == 2) { if (pro) MRS_SG(2, 1); else MRS_SG(2, 0); return check_launch("skinny_gemm_kernel"); }
    }
    if (pro) MRS_SG(0, 1); else MRS_SG(0, 0);
#undef MRS_SG
    return check_launch("skinny_gemm_kernel");
}

int skinny_max_rows() {
    static const int v = [] { const char *e = getenv("MRS_SKINNY_MAX_ROWS"); const int n = e ? atoi(e) : 128; return n < 1 ? 1 : (n > 1024 ? 1024 : n); }();
    return v;
}

bool skinny_gemm_ok(int dtype, int M, int N, int K, int64_t lda, const void *A, const void *Wt) {
    if (dtype == MRS_F32)   // row-wise route only: one to four rows, K a multiple of 32 lanes x 4 elements, rows that fit in LDS
        return M >= 1 && M <= 4 && N >= 1 && K >= 128 && K % 128 == 0 && (int64_t)K * 16 <= 48 * 1024 && lda % 4 == 0 && aligned(A, 16) &&
               aligned(Wt, 16) && !no_rowwise_route();
    return (dtype == MRS_BF16 || dtype == MRS_F16) && M >= 1 && M <= skinny_max_rows() && N >= 1 && K >= 32 && K % 32 == 0 && lda % 8 == 0 &&
           aligned(A, 16) && aligned(Wt, 16);
}

int launch_skinny_gemm(hipStream_t st, int dtype, void *C, int out_f32, int64_t ldc, const void *A, int64_t lda, const void *Wt,
                       int M, int N, int K, const SkinnyEpi &ep) {
    if (!skinny_gemm_ok(dtype, M, N, K, lda, A, Wt))
        return fail(MRS_E_SHAPE, "skinny gemm: needs 16-bit storage with 1 <= M <= 128, K %% 32 == 0, lda %% 8 == 0, or f32 storage with M <= 4, "
                                 "K %% 128 == 0, lda %% 4 == 0; 16-byte aligned A and Wt (got dtype=%d M=%d N=%d K=%d lda=%lld)", dtype, M, N, K,
                    (long long)lda);
    if (ep.mode == 1 && (ep.dc < 1 || ep.dc > kMaxConvTaps || ep.di < 1 || ep.di > N || !ep.conv_state || !ep.conv_w || !ep.conv_b || !ep.u))
        return fail(MRS_E_SHAPE, "skinny gemm: bad in_proj epilogue (di=%d dc=%d)", ep.di, ep.dc);
    if (ep.mode == 1 && ep.xw && (ep.xd < 1 || ep.di % 16 != 0 || !ep.xpart))
        return fail(MRS_E_SHAPE, "skinny gemm: bad folded x_proj (M=%d xd=%d di=%d)", M, ep.xd, ep.di);
    if (ep.mode == 2 && (!ep.residual || !ep.partials || ep.n_partials != (N + 15) / 16 || (ep.next_norm_w && !ep.prenorm)))
        return fail(MRS_E_SHAPE, "skinny gemm: bad out_proj epilogue (n_partials=%d, column tiles=%d)", ep.n_partials, (N + 15) / 16);
    if (ep.row_scale && (!ep.partials || ep.n_partials < 1))
        return fail(MRS_E_SHAPE, "skinny gemm: row scale without partial sums");
    if (dtype == MRS_F32) return launch_skinny_t<float, float>(st, (float *)C, ldc, (const float *)A, lda, (const float *)Wt, M, N, K, ep);
    if (dtype == MRS_BF16) {
        if (out_f32) return launch_skinny_t<bf16_t, float>(st, (float *)C, ldc, (const bf16_t *)A, lda, (const bf16_t *)Wt, M, N, K, ep);
        return launch_skinny_t<bf16_t, bf16_t>(st, (bf16_t *)C, ldc, (const bf16_t *)A, lda, (const bf16_t *)Wt, M, N, K, ep);
    }
    if (out_f32) return launch_skinny_t<f16_t, float>(st, (float *)C, ldc, (const f16_t *)A, lda, (const f16_t *)Wt, M, N, K, ep);
    return launch_skinny_t<f16_t, f16_t>(st, (f16_t *)C, ldc, (const f16_t *)A, lda, (const f16_t *)Wt, M, N, K, ep);
}

int launch_prenorm_rows(hipStream_t st, int dtype, float *partials, int n_partials, void *prenorm, const float *x, float *copy_to,
                        const float *w, int M, int K, int a_mt) {
    if (dtype == MRS_BF16) hipLaunchKernelGGL((prenorm_rows_kernel<bf16_t>), dim3((unsigned)M), dim3(256), 0, st, partials, n_partials, (bf16_t *)prenorm, x, copy_to, w, K, a_mt);
    else if (dtype == MRS_F16) hipLaunchKernelGGL((prenorm_rows_kernel<f16_t>), dim3((unsigned)M), dim3(256), 0, st, partials, n_partials, (f16_t *)prenorm, x, copy_to, w, K, a_mt);
    else hipLaunchKernelGGL((prenorm_rows_kernel<float>), dim3((unsigned)M), dim3(256), 0, st, partials, n_partials, (float *)prenorm, x, copy_to, w, K, a_mt);
    return check_launch("prenorm_rows_kernel");
}

bool dt_proj_softplus_ok(int dtype, int di, int dr, int64_t xs, const void *delta, const void *dt_in, const void *wt) {
    return (dtype == MRS_BF16 || dtype == MRS_F16) && di % 64 == 0 && dr >= 8 && dr % 8 == 0 && dr <= 256 && xs % 8 == 0 && xs >= dr &&
           aligned(delta, 16) && aligned(dt_in, 16) && aligned(wt, 16);
}

int launch_dt_proj_softplus(hipStream_t st, int dtype, void *delta, const void *dt_in, int64_t xs, const void *wt, const float *bias,
                            int64_t rows, int di, int dr) {
    if (!dt_proj_softplus_ok(dtype, di, dr, xs, delta, dt_in, wt))
        return fail(MRS_E_SHAPE, "dt_proj+softplus: needs 16-bit storage, d_inner a multiple of 64, dt_rank and the row stride multiples of 8, 16-byte aligned operands");
    if (rows < 1) return fail(MRS_E_SHAPE, "dt_proj+softplus: rows=%lld", (long long)rows);
    // About eight workgroups per compute unit, each walking several row tiles -- as many as its neighbours where the tile
    // count allows: the launch takes as long as the workgroup with the most tiles (2.8b shape, 256 row tiles over 40 column
    // blocks: 32 workgroups per block with 8 tiles each 78.5 us, 52 with 4 or 5 tiles 85.7 us).
    const int ks = (dr + 31) / 32;
    // columns per workgroup (every block is whole: the stores carry no column test): 64 with the weight in registers; with
    // the weight in LDS 128 where d_inner allows
    const bool wlds = ks >= 4;
    const int ct = wlds && di % 128 == 0 ? 8 : 4;
    const int64_t n_tiles = (rows + 63) / 64;
    const int gx = (di + 16 * ct - 1) / (16 * ct);
    int64_t gy = std::max<int64_t>(1, std::min<int64_t>(n_tiles, (2048 + gx - 1) / gx));
    for (int64_t d = gy; 2 * d > gy; d--)
        if (n_tiles % d == 0) { gy = d; break; }
    const dim3 grid((unsigned)gx, (unsigned)gy), block(256);
#define MRS_DTP_CT(T_, KS_, CT_) hipLaunchKernelGGL((dt_proj_softplus_kernel<T_, KS_, CT_, (KS_ >= 4)>), grid, block, 0, st, (T_ *)delta, (const T_ *)dt_in, xs, (const T_ *)wt, bias, rows, di, dr)
#define MRS_DTP(T_, KS_)                                                    \
    do {                                                                    \
        if constexpr (KS_ >= 4) { if (ct == 8) MRS_DTP_CT(T_, KS_, 8); else MRS_DTP_CT(T_, KS_, 4); } \
        else MRS_DTP_CT(T_, KS_, 4);                                        \
    } while (0)
#define MRS_DTP_KS(T_)                                      \
    switch (ks) {                                           \
        case 1: MRS_DTP(T_, 1); break;                      \
        case 2: MRS_DTP(T_, 2); break;                      \
        case 3: MRS_DTP(T_, 3); break;                      \
        case 4: MRS_DTP(T_, 4); break;                      \
        case 5: case 6: MRS_DTP(T_, 6); break;              \
        default: MRS_DTP(T_, 8); break;                     \
    }
    if (dtype == MRS_BF16) { MRS_DTP_KS(bf16_t) } else { MRS_DTP_KS(f16_t) }
#undef MRS_DTP_KS
#undef MRS_DTP
#undef MRS_DTP_CT
    return check_launch("dt_proj_softplus_kernel");
}

int launch_transpose(hipStream_t st, int dtype, void *Wt, const void *W, int K, int N) {
    const dim3 grid((unsigned)((N + 31) / 32), (unsigned)((K + 31) / 32)), block(256);
    if (dtype == MRS_F32) hipLaunchKernelGGL((transpose_kernel<float>), grid, block, 0, st, (float *)Wt, (const float *)W, K, N);
    else hipLaunchKernelGGL((transpose_kernel<uint16_t>), grid, block, 0, st, (uint16_t *)Wt, (const uint16_t *)W, K, N);
    return check_launch("transpose_kernel");
}

}  // namespace mrs

using namespace mrs;

extern "C" int mrs_gemm_skinny(void *stream, int dtype, void *C, int out_f32, int64_t ldc, const void *A, int64_t lda,
                               const void *Wt, int M, int N, int K) {
    if (!C || !A || !Wt) return fail(MRS_E_NULL, "mrs_gemm_skinny: null pointer");
    if (ldc < N) return fail(MRS_E_SHAPE, "mrs_gemm_skinny: ldc=%lld < N=%d", (long long)ldc, N);
    if (lda < K) return fail(MRS_E_SHAPE, "mrs_gemm_skinny: lda=%lld < K=%d", (long long)lda, K);
    SkinnyEpi ep = {};
    return launch_skinny_gemm(as_stream(stream), dtype, C, out_f32, ldc, A, lda, Wt, M, N, K, ep);
}

extern "C" int mrs_transpose(void *stream, int dtype, void *Wt, const void *W, int K, int N) {
    if (!Wt || !W) return fail(MRS_E_NULL, "mrs_transpose: null pointer");
    if (dtype != MRS_F32 && dtype != MRS_F16 && dtype != MRS_BF16) return fail(MRS_E_DTYPE, "mrs_transpose: dtype %d", dtype);
    if (K < 1 || N < 1) return fail(MRS_E_SHAPE, "mrs_transpose: K=%d N=%d", K, N);
    return launch_transpose(as_stream(stream), dtype, Wt, W, K, N);
}
