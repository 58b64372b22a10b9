// Decode GEMM for wide models: C[M,N] = A[M,K] . W[K,N] with up to 64 rows (the batch; the decode chain comes here from 3 rows) and a weight of megabytes
// (in_proj of the 2.8b shape: 2560 x 10240, 52 MB), 16-bit operands, f32 accumulate on the matrix cores.
//
// The reference sends these products to the vendor GEMM (cuBLAS call sites src/mamba_ssm/gpu/blas.rs:1138-1163).  At
// this size the product is one pass over the weight and nothing else, so the kernel is built around that stream:
//   * the weight is kept TILED: the 16 columns x 32 k of one v_mfma_f32_16x16x32 B operand are 1 KB of consecutive
//     memory in lane order (lane l: column l % 16, k = 8 (l / 16) .. +7), the k-steps of a column tile follow each other.
//     A wave's load instruction then fetches one whole kilobyte and a wave streams a contiguous region -- with the
//     row-major transposed copy the same instruction touches sixteen 64-byte pieces 2 K bytes apart (measured on the
//     2.8b in_proj at 16 rows: 18.5 us tiled, 21.8 us row-major, the rest of the kernel being equal);
//   * a workgroup owns 16 NT output columns (NT column tiles, up to three) over ALL of K and all rows.  Two or four of its eight
//     waves stream the operands, wave w taking k-steps w, w + WS, ..., so every weight byte is requested once, by one
//     wave, and no sum leaves the workgroup: the waves' partial tiles meet in LDS (splitting K over workgroups instead, with
//     the slices meeting in memory behind an arrival counter, cost 4-6 us of store / count / reload round trips at the
//     end of a 12 us stream).  The other waves only share the epilogue: more streaming waves put more requests in
//     front of the memory system at once and the stream gets slower, fewer epilogue threads make the end of the kernel
//     a serial walk over the tile;
//   * a streaming wave keeps R k-steps of operand pieces requested ahead in registers, weight tiles and activation
//     pieces of the same k-step side by side in the order they are used.  The operands come through buffer resources
//     that end where K ends (a piece past the end is zeros and no traffic), so the loop has no tail and no branch, and
//     scheduling barriers keep every refill right behind its use: the compiler then waits for exactly the oldest
//     k-step (vmcnt = everything younger) -- with conditional loads it waited for all of them every round;
//   * the activation operand is read in the same tiled order (16 rows x 32 k = 1 KB in lane order, tiled_a_index) when
//     its producer wrote it so (the decode chain does: prenorm, the out_proj epilogue and the step kernel write
//     in_proj's and out_proj's operands tiled).  Row-major rows work too, but a load of sixteen 64-byte row pieces
//     costs the L1 sixty-four tag look-ups where a tile costs eight (in_proj at 64 rows: 24 us tiled, 38 us row-major);
//   * the epilogues are those of gemm_skinny.hip (plain store, in_proj's conv step + SiLU, out_proj's residual add with
//     the row's sums of squares), one result element per thread and pass: element (row ml, column nl) of a 16 x 16 tile
//     sits in lane 16 (ml / 4) + nl, register ml % 4 of the accumulator.  The epilogue operands of all of a thread's
//     elements are requested together behind the first operand requests; the rows' scales are formed by the waves
//     that do not stream.
#include "common.hpp"
#include "mfma_tiles.hpp"
#include <stdlib.h>
#include <algorithm>

namespace mrs {
namespace {

constexpr int kTiledThreads = 512;   // eight waves per workgroup: WS of them stream the operands, all of them run the epilogue

template <typename T, int MT, int NT, int R, int WS = 8>
__global__ __launch_bounds__(kTiledThreads) void tiled_gemm_kernel(void *__restrict__ Cv, int out_f32, int64_t ldc, const T *__restrict__ A,
                                                                   int64_t lda, const T *__restrict__ Wp, int M, int N, int K, SkinnyEpi ep) {
    constexpr int kPark = WS;   // partial tiles that meet in LDS, one per streaming wave
    __shared__ v4f red[kPark][MT * NT][kWave];
    __shared__ float inv_s[16 * MT];
    const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, lr = l & 15, lg = l >> 4;
    const int nks = K >> 5, per = (nks + WS - 1) / WS;
    const int ntiles = (N + 15) >> 4;
    // Operands through buffer resources that end where K ends: a piece past the end arrives as zeros and costs no memory
    // traffic, so the loop below has no tail and no branch -- every wave runs the same ceil(per / R) rounds and the
    // compiler can count the loads in flight exactly.
    __amdgpu_buffer_rsrc_t wres[NT];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        const T *base = Wp + (int64_t)min((int)blockIdx.x * NT + nt, ntiles - 1) * nks * 512;
        wres[nt] = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(base), 0, nks * 1024, 0x00020000);
    }
    // activation rows, row-major: the whole matrix is the range (a k-step past K meets zero weights; past the last row's
    // end it is zero itself), rows past M repeat the last one.  Tiled (ep.a_tiled): [k-step][row tile][lane][8], the A
    // operand in lane order like the weight, 16 MT rows.
    const bool a_tiled = ep.a_tiled != 0;
    const int a_records = a_tiled ? nks * MT * 1024 : (int)((((int64_t)(M - 1) * lda + K) * (int64_t)sizeof(T)));
    const __amdgpu_buffer_rsrc_t ares = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(A), 0, a_records, 0x00020000);
    unsigned aoff[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
        aoff[mt] = a_tiled ? (unsigned)(mt * 1024 + 16 * l) : (unsigned)(((int64_t)min(16 * mt + lr, M - 1) * lda + 8 * lg) * (int64_t)sizeof(T));
    const unsigned astep = a_tiled ? (unsigned)MT * 1024u : 64u;
    const unsigned woff = 16u * (unsigned)l;
    auto ldw = [&](int nt, int s_) {
        return __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(wres[nt], woff, 1024u * (unsigned)(w + WS * s_), 0));
    };
    auto lda_ = [&](int mt, int s_) {
        const int ks = w + WS * s_;
        const unsigned so = ks < nks ? astep * (unsigned)ks : (unsigned)a_records;
        return __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(ares, aoff[mt], so, 0));
    };
    // Epilogue work is spread over all threads: element e = tid + (threads) j of the workgroup's MT NT tiles of 256 -- tile
    // e / 256, row (e % 256) / 16 and column e % 16 of it -- so sixteen consecutive lanes share a row.
    constexpr int kTiles = MT * NT;
    constexpr int EP = (kTiles * 256 + kTiledThreads - 1) / kTiledThreads;
    // The operands of an element's epilogue (conv window, taps and bias; or residual and next norm weight) are requested
    // for all of a thread's elements at once, right behind the first operand requests (the conv windows of a decode step
    // are cold: fetched inside the element loop they would be a memory round trip per element, behind the stream one
    // round trip at the end of the kernel; a workgroup per compute unit has the registers to hold them).
    float4 pf_win[EP], pf_tap[EP];
    float pf_x[EP], pf_y[EP];
    auto request_epilogue = [&]() {
        // Four loads per element, issued on every path with no branch around them: the addresses are chosen by selects (a
        // clamped row / column where the element lies outside the result, the activation operand's first bytes where the
        // epilogue has no such operand).  A value that is a load on one path and something else on another has to be copied
        // into place once the load is back, and the wait for that copy sat in front of the operand stream -- a memory round
        // trip for the cold conv windows before the first weight request.
        const bool conv4 = ep.mode == 1 && ep.dc == 4, resid = ep.mode == 2;
        const float4 *dummy4 = reinterpret_cast<const float4 *>(A);
        const float *dummy = reinterpret_cast<const float *>(A);
#pragma unroll
        for (int j = 0; j < EP; j++) {
            const int e = tid + kTiledThreads * j, tile = min(e >> 8, kTiles - 1);
            const int row = min(16 * (tile / NT) + ((e >> 4) & 15), M - 1), col = min(16 * ((int)blockIdx.x * NT + tile % NT) + (e & 15), N - 1);
            const int cc = conv4 ? min(col, ep.di - 1) : 0;
            const float4 *pw = conv4 ? reinterpret_cast<const float4 *>(ep.conv_state + ((int64_t)row * ep.di + cc) * 4) : dummy4;
            const float4 *pt = conv4 ? reinterpret_cast<const float4 *>(ep.conv_w + (int64_t)cc * 4) : dummy4;
            const float *px = conv4 ? ep.conv_b + cc : (resid ? ep.residual + (int64_t)row * N + col : dummy);
            const float *py = (resid && ep.next_norm_w) ? ep.next_norm_w + col : dummy;
            pf_win[j] = *pw; pf_tap[j] = *pt; pf_x[j] = *px; pf_y[j] = *py;
        }
    };
    // waves 0 .. WS-1 stream the operands (wave w takes k-steps w, w + WS, ...); the others only share the epilogue
    const bool streams = w < WS;
    uint4 wr[R][NT], ar[R][MT];
    if (streams) {
#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++) wr[r][nt] = ldw(nt, r);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) ar[r][mt] = lda_(mt, r);
            __builtin_amdgcn_sched_barrier(0);   // requested in the order of use, as in the loop (the wait counts of its first round follow this order)
        }
    }
    request_epilogue();   // behind the first operand requests: loads come back in the order they were issued
    // RMSNorm folded around the product (gemm_skinny.hip): 1/rms of each row from its partial sums of squares, by the
    // waves that do not stream (the streaming waves entered their loop 1.3 us later when they shared this).  Sixteen
    // lanes share a row; its partial sums (up to 256 of them, a multiple of four) are fetched as 16-byte pieces, all of a
    // row's at once -- summed one load at a time in a loop they were ten L2 round trips in a row.
    static_assert(WS <= 4, "at least four waves beside the streaming ones");
    if (ep.row_scale && !streams) {
        constexpr int kHelpers = kTiledThreads - 64 * WS;
        const int ht = tid - 64 * WS;
        const bool ps_fast = ep.n_partials % 4 == 0 && ep.n_partials <= 256;
        for (int r = ht >> 4; r < 16 * MT; r += kHelpers / 16) {
            const float *pp = ep.partials + (int64_t)min(r, M - 1) * ep.n_partials;
            float ss = 0.0f;
            if (ps_fast) {
                float4 ps[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int p4 = 4 * ((ht & 15) + 16 * q);
                    ps[q] = p4 < ep.n_partials ? *reinterpret_cast<const float4 *>(pp + p4) : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int q = 0; q < 4; q++) ss += (ps[q].x + ps[q].y) + (ps[q].z + ps[q].w);
            } else {
                for (int p_ = ht & 15; p_ < ep.n_partials; p_ += 16) ss += pp[p_];
            }
#pragma unroll
            for (int m = 8; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
            float rms = sqrtf(ss / (float)K + ep.eps);
            if (!isfinite(rms) || rms < 1e-20f) rms = 1.0f;
            if ((ht & 15) == 0) inv_s[r] = 1.0f / rms;
        }
    }
    v4f acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++) acc[mt][nt] = (v4f){0.f, 0.f, 0.f, 0.f};
    for (int kb = 0; streams && kb < per; kb += R) {
#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
#pragma unroll
                for (int mt = 0; mt < MT; mt++) acc[mt][nt] = Mma32<T>::mma(ar[r][mt], wr[r][nt], acc[mt][nt]);
#pragma unroll
            for (int nt = 0; nt < NT; nt++) wr[r][nt] = ldw(nt, kb + r + R);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) ar[r][mt] = lda_(mt, kb + r + R);
            __builtin_amdgcn_sched_barrier(0);   // keep each refill right behind its use: the scheduler would gather the loads at the end of the round
        }
    }
    // the K ranges meet in LDS: every streaming wave parks its tiles, and the thread that owns an element adds them in
    // wave order (one fixed order of additions, one barrier)
    if (streams) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int nt = 0; nt < NT; nt++) red[w][mt * NT + nt][l] = acc[mt][nt];
    }
    lds_barrier();
    T *C = reinterpret_cast<T *>(Cv);
    float *Cf = reinterpret_cast<float *>(Cv);
#pragma unroll
    for (int j = 0; j < EP; j++) {
        const int e = tid + kTiledThreads * j;
        const int tile = e >> 8;                        // the same for a whole wave
        if (tile >= kTiles) break;
        // element (ml, nl) of a 16 x 16 tile sits in lane 16 (ml / 4) + nl, register ml % 4 of the accumulator
        const int ml = (e >> 4) & 15, nl = e & 15, lane = (ml >> 2) * 16 + nl, i = ml & 3;
        float s = red[0][tile][lane][i];
#pragma unroll
        for (int q = 1; q < kPark; q++) s += red[q][tile][lane][i];
        const int ctile = (int)blockIdx.x * NT + tile % NT;
        const int row = 16 * (tile / NT) + ml, col = 16 * ctile + nl;
        const bool valid = row < M && col < N;
        if (ep.row_scale) s *= inv_s[row];
        if (ep.mode == 2) {
            // out_proj: residual += out (rounded to the storage type as the stored projection would be); the row's sum of
            // squares over these 16 columns and the pre-scaled operand of the next layer's in_proj
            float sq = 0.0f;
            if (valid) {
                const T orr = (T)s;
                const float res_old = pf_x[j];
                const float nw = ep.next_norm_w ? pf_y[j] : 0.0f;
                const float rn = res_old + Store<T>::ld(&orr);
                ep.residual[(int64_t)row * N + col] = rn;
                sq = rn * rn;
                if (ep.next_norm_w)
                    Store<T>::st(reinterpret_cast<T *>(ep.prenorm) + (ep.prenorm_mt ? tiled_a_index(row, col, ep.prenorm_mt) : (int64_t)row * N + col), rn * nw);
            }
#pragma unroll
            for (int m = 8; m >= 1; m >>= 1) sq += __shfl_xor(sq, m, kWave);
            if (nl == 0 && row < M && 16 * ctile < N) ep.partials[(int64_t)row * ep.n_partials + ctile] = sq;
        } else if (!valid) {
        } else if (ep.mode == 1 && col < ep.di) {
            // conv step on the value as in_proj would have stored it (conv1d_step_forward_silu, kernels/conv1d.cu:85-115)
            const T xr = (T)s;
            const float xnew = Store<T>::ld(&xr);
            float *st = ep.conv_state + ((int64_t)row * ep.di + col) * ep.dc;
            const float *cw = ep.conv_w + (int64_t)col * ep.dc;
            float o;
            if (ep.dc == 4) {   // window and taps are one aligned 16-byte vector each
                const float4 win = pf_win[j];
                const float4 tap = pf_tap[j];
                o = pf_x[j];
                o = fmaf(win.y, tap.x, o); o = fmaf(win.z, tap.y, o); o = fmaf(win.w, tap.z, o); o = fmaf(xnew, tap.w, o);
                *reinterpret_cast<float4 *>(st) = make_float4(win.y, win.z, win.w, xnew);
            } else {
                o = ep.conv_b[col];
                for (int k = 0; k < ep.dc; k++) {
                    const float wk = (k + 1 < ep.dc) ? st[k + 1] : xnew;
                    o = fmaf(wk, cw[k], o);
                    st[k] = wk;
                }
            }
            const T ur = (T)silu(o);
            reinterpret_cast<T *>(ep.u)[(int64_t)row * ep.di + col] = ur;
            if (ep.u_tiled) reinterpret_cast<T *>(ep.u_tiled)[tiled_a_index(row, col, ep.u_tiled_mt)] = ur;   // x_proj's operand
        } else if (out_f32) {
            Cf[(int64_t)row * ldc + col] = s;
        } else {
            Store<T>::st(C + (int64_t)row * ldc + col, s);
        }
    }
}

// Wp[column tile][k-step][lane][8] from the transposed weight Wt[N][K]; columns past N are zero
template <typename T>
__global__ __launch_bounds__(256) void tile_weight_kernel(uint4 *__restrict__ Wp, const T *__restrict__ Wt, int N, int K, int64_t pieces) {
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= pieces) return;
    const int lane = (int)(p & 63), nks = K >> 5;
    const int64_t t = p >> 6;
    const int ks = (int)(t % nks);
    const int col = (int)(t / nks) * 16 + (lane & 15);
    Wp[p] = col < N ? *reinterpret_cast<const uint4 *>(Wt + (int64_t)col * K + 32 * ks + 8 * (lane >> 4)) : make_uint4(0, 0, 0, 0);
}

template <typename T>
int launch_tiled_t(hipStream_t st, void *C, int out_f32, int64_t ldc, const T *A, int64_t lda, const T *Wp, int M, int N, int K,
                   const SkinnyEpi &ep) {
    const int mt = (M + 15) / 16;
    const int ntiles = (N + 15) / 16;
    // Column tiles per workgroup.  A compute unit keeps about 64 KB of requests in flight whatever runs on it (measured
    // with time stamps per workgroup: two workgroups sharing a unit each take twice as long), so a launch takes as long
    // as the unit with the most tiles: ceil(workgroups / 256) NT of them.  NT is the count of up to three that makes
    // this smallest, the larger on a tie (fewer workgroups read the activation operand).  in_proj of the 2.8b shape,
    // 640 tiles: 214 workgroups of three tiles -- with two tiles 320 workgroups, 64 units run two of them one after the
    // other while the rest of the chip idles (alone, with a plain store, 64 rows: 22.6 us against 15.4 us; 16 rows, one
    // tile: 12.9 against 11.4).
    int nt = 1, worst = 1 << 30;
    for (int c = 1; c <= 3; c++) {
        const int wgs = (ntiles + c - 1) / c, load = (wgs + 255) / 256 * c;
        if (load <= worst) { worst = load; nt = c; }
    }
    // Streaming waves WS (they split K) and k-steps R each keeps requested ahead: WS R (NT + MT) KB in flight per
    // workgroup, 48 to 64 of them -- more only queues in front of the unit's memory pipeline (alone, with a plain
    // store, in_proj at 16 rows and one tile takes 13.7 us with one streaming wave and 18.3 us with eight).  In the
    // 2.8b-shape decode chain, per step with 1 / 2 / 4 / 8 streaming waves: 16 rows 2.85 / 2.75 / 2.65 / 2.72 ms,
    // 32 rows 3.48 / 3.35 / 3.44 / 3.62, 64 rows 5.29 / 4.77 / 4.81 / 4.92.
    const dim3 grid((unsigned)((ntiles + nt - 1) / nt)), block(kTiledThreads);
#define MRS_TG(MT_, NT_, R_, W_) \
    hipLaunchKernelGGL((tiled_gemm_kernel<T, MT_, NT_, R_, W_>), grid, block, 0, st, C, out_f32, ldc, A, lda, Wp, M, N, K, ep)
    switch (mt * 10 + nt) {
        case 11: MRS_TG(1, 1, 10, 4); break;
        case 12: MRS_TG(1, 2, 5, 4); break;
        case 13: MRS_TG(1, 3, 4, 4); break;
        case 21: MRS_TG(2, 1, 8, 2); break;
        case 22: MRS_TG(2, 2, 6, 2); break;
        case 23: MRS_TG(2, 3, 3, 4); break;
        case 31: MRS_TG(3, 1, 6, 2); break;
        case 32: MRS_TG(3, 2, 5, 2); break;
        case 33: MRS_TG(3, 3, 5, 2); break;
        case 41: MRS_TG(4, 1, 5, 2); break;
        case 42: MRS_TG(4, 2, 4, 2); break;
        default: MRS_TG(4, 3, 2, 4); break;
    }
#undef MRS_TG
    return check_launch("tiled_gemm_kernel");
}

}  // namespace

bool tiled_gemm_ok(int dtype, int M, int N, int K, int64_t lda, const void *A, const void *Wp) {
    return (dtype == MRS_BF16 || dtype == MRS_F16) && M >= 1 && M <= 64 && N >= 1 && K >= 32 && K % 32 == 0 && lda % 8 == 0 && aligned(A, 16) &&
           aligned(Wp, 16);
}

size_t tiled_weight_elems(int N, int K) { return (size_t)((N + 15) / 16) * 16 * (size_t)K; }

int launch_tile_weight(hipStream_t st, int dtype, void *Wp, const void *Wt, int N, int K) {
    if ((dtype != MRS_BF16 && dtype != MRS_F16) || K < 32 || K % 32 != 0 || N < 1 || !aligned(Wp, 16) || !aligned(Wt, 16))
        return fail(MRS_E_SHAPE, "tile weight: 16-bit storage, K %% 32 == 0, 16-byte aligned operands (dtype=%d N=%d K=%d)", dtype, N, K);
    const int64_t pieces = (int64_t)((N + 15) / 16) * (K >> 5) * 64;
    hipLaunchKernelGGL((tile_weight_kernel<uint16_t>), dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (uint4 *)Wp, (const uint16_t *)Wt, N, K, pieces);
    return check_launch("tile_weight_kernel");
}

int launch_tiled_gemm(hipStream_t st, int dtype, void *C, int out_f32, int64_t ldc, const void *A, int64_t lda, const void *Wp, int M,
                      int N, int K, const SkinnyEpi &ep) {
    if (!tiled_gemm_ok(dtype, M, N, K, lda, A, Wp))
        return fail(MRS_E_SHAPE, "tiled gemm: needs 16-bit storage, 1 <= M <= 64, K %% 32 == 0, lda %% 8 == 0, 16-byte aligned A and weight "
                                 "(got dtype=%d M=%d N=%d K=%d lda=%lld)", dtype, M, N, K, (long long)lda);
    if (ep.xw || (ep.mode == 0 && ep.ksplit > 1) || ep.mode < 0 || ep.mode > 2)
        return fail(MRS_E_SHAPE, "tiled gemm: the x_proj shares ride on the 16-row tiles of the row-major route only");
    if (dtype == MRS_BF16) return launch_tiled_t<bf16_t>(st, C, out_f32, ldc, (const bf16_t *)A, lda, (const bf16_t *)Wp, M, N, K, ep);
    return launch_tiled_t<f16_t>(st, C, out_f32, ldc, (const f16_t *)A, lda, (const f16_t *)Wp, M, N, K, ep);
}

}  // namespace mrs

using namespace mrs;

extern "C" size_t mrs_tiled_weight_bytes(int dtype, int N, int K) {
    if ((dtype != MRS_BF16 && dtype != MRS_F16) || N < 1 || K < 32 || K % 32 != 0) return 0;
    return tiled_weight_elems(N, K) * 2;
}

extern "C" int mrs_tile_weight(void *stream, int dtype, void *Wp, const void *Wt, int N, int K) {
    if (!Wp || !Wt) return fail(MRS_E_NULL, "mrs_tile_weight: null pointer");
    return launch_tile_weight(as_stream(stream), dtype, Wp, Wt, N, K);
}

extern "C" int mrs_gemm_tiled(void *stream, int dtype, void *C, int out_f32, int64_t ldc, const void *A, int64_t lda, const void *Wp,
                              int M, int N, int K) {
    if (!C || !A || !Wp) return fail(MRS_E_NULL, "mrs_gemm_tiled: null pointer");
    if (ldc < N) return fail(MRS_E_SHAPE, "mrs_gemm_tiled: ldc=%lld < N=%d", (long long)ldc, N);
    if (lda < K) return fail(MRS_E_SHAPE, "mrs_gemm_tiled: lda=%lld < K=%d", (long long)lda, K);
    SkinnyEpi ep = {};
    // a weight of 16 MB or more on the column-tile kernel (up to 64 rows), a smaller one on the 16 x 16 tiles of
    // gemm_skinny.hip reading the same tiled weight (up to 128 rows): the split the decode chain makes
    if ((int64_t)N * K * 2 >= ((int64_t)16 << 20) && M <= 64) return launch_tiled_gemm(as_stream(stream), dtype, C, out_f32, ldc, A, lda, Wp, M, N, K, ep);
    if (dtype != MRS_BF16 && dtype != MRS_F16) return fail(MRS_E_DTYPE, "mrs_gemm_tiled: 16-bit storage only");
    ep.w_tiled = 1;
    return launch_skinny_gemm(as_stream(stream), dtype, C, out_f32, ldc, A, lda, Wp, M, N, K, ep);
}
