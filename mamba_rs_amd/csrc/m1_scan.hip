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
#include <stdlib.h>
#include <mutex>

namespace mrs {

constexpr int kNPL = 16;  // state entries held per lane

// Raw (unconverted) element types, so loads can be issued well ahead of the arithmetic that widens and uses them.
template <typename T> struct RawElem { using type = uint16_t; };
template <> struct RawElem<float> { using type = float; };
__device__ __forceinline__ float widen(float v, const float *) { return v; }
__device__ __forceinline__ float widen(uint16_t v, const bf16_t *) { return __uint_as_float((uint32_t)v << 16); }
__device__ __forceinline__ float widen(uint16_t v, const f16_t *) { return (float)__builtin_bit_cast(_Float16, v); }
template <typename T> __device__ __forceinline__ typename RawElem<T>::type raw_ld(const T *p) {
    return *reinterpret_cast<const typename RawElem<T>::type *>(p);
}

// ---------------------------------------------------------------------------
// Generic sequential kernel.  LPC lanes share one channel, lane g of the group
// owning states n in [16g, 16g+16); any d_state <= 16*LPC, any d_inner.
// One wave per (batch row, tile of 64/LPC channels); time runs serially.
// A wave alone on its SIMD has nothing to hide a memory round trip behind, so
// time is walked in blocks of 16 steps: the operands of the next block are
// requested (raw, into registers) before the current block is computed --
// delta / u / gate per lane, the block's B and C rows spread over the lanes and
// handed round through LDS.  (One request per step was 2.5 us per step.)
// ---------------------------------------------------------------------------
constexpr int kSeqBlock = 16;
template <typename T, int LPC, bool S4D, int GATE>
__global__ __launch_bounds__(kWave) void ssm_scan_seq_kernel(
    float *__restrict__ h, T *__restrict__ y, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, const T *__restrict__ Cm, int64_t bc_stride,
    const float *__restrict__ a_neg, const float *__restrict__ Dp, const T *__restrict__ gate,
    int64_t gate_stride, int Tlen, int di, int ds, int tiles) {
    using raw_t = typename RawElem<T>::type;
    constexpr int CPW = kWave / LPC;
    constexpr int W = kNPL * LPC;                      // padded row width in LDS
    constexpr int NBC = kSeqBlock * W / kWave;         // B (and C) elements of a block per lane
    __shared__ alignas(16) raw_t bc[2][2][kSeqBlock * W];   // [buffer][B | C][step][n]
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

    raw_t rd[kSeqBlock], ru[kSeqBlock], rg[kSeqBlock], nd[kSeqBlock], nu[kSeqBlock], ng[kSeqBlock];
    raw_t nB[NBC], nC[NBC];
    auto request = [&](raw_t (&xd)[kSeqBlock], raw_t (&xu)[kSeqBlock], raw_t (&xg)[kSeqBlock], int tb) {
#pragma unroll
        for (int s = 0; s < kSeqBlock; s++) {
            const int64_t row = row0 + min(tb + s, Tlen - 1);   // past the end: the last row again, computed and dropped
            xd[s] = raw_ld(delta + row * di + dd);
            xu[s] = raw_ld(u + row * di + dd);
            if (GATE) xg[s] = raw_ld(gate + row * gate_stride + dd);
        }
#pragma unroll
        for (int i = 0; i < NBC; i++) {
            const int e = lane + kWave * i, s = e / W, n = e - s * W;
            const int64_t row = row0 + min(tb + s, Tlen - 1);
            const int nn = min(n, ds - 1);                      // padding columns: an in-range element, never used
            nB[i] = raw_ld(Bm + row * bc_stride + nn);
            nC[i] = raw_ld(Cm + row * bc_stride + nn);
        }
    };
    auto publish = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NBC; i++) {
            bc[buf][0][lane + kWave * i] = nB[i];
            bc[buf][1][lane + kWave * i] = nC[i];
        }
    };
    request(rd, ru, rg, 0);
    publish(0);
    int buf = 0;
    for (int tb = 0; tb < Tlen; tb += kSeqBlock, buf ^= 1) {
        lds_barrier();   // the block's rows are in LDS (one wave: orders its own LDS traffic, global loads stay in flight)
        if (tb + kSeqBlock < Tlen) request(nd, nu, ng, tb + kSeqBlock);
#pragma unroll
        for (int s = 0; s < kSeqBlock; s++) {
            const int t = tb + s;
            if (t < Tlen) {
                const float dl = widen(rd[s], (const T *)nullptr);
                const float uu = widen(ru[s], (const T *)nullptr);
                const float du = dl * uu;
                float acc = (g == 0) ? Dd * uu : 0.0f;
                // the lane's 16 B and 16 C values of this step as whole 16-byte LDS reads (read unconditionally, masked
                // below: a conditional read per element became a branch and a wait per element)
                struct alignas(16) RawRow { raw_t v[kNPL]; };
                const RawRow Br = *reinterpret_cast<const RawRow *>(&bc[buf][0][s * W + n0]);
                const RawRow Cr = *reinterpret_cast<const RawRow *>(&bc[buf][1][s * W + n0]);
                float pw = 0.0f, p1 = 0.0f;
                if (S4D) {
                    p1 = fast_exp2(dl * a20);
                    pw = (LPC == 1) ? p1 : fast_exp2(dl * a20 * (float)(n0 + 1));
                }
#pragma unroll
                for (int j = 0; j < kNPL; j++) {
                    const bool nv = (n0 + j) < ds;
                    const float Bn = nv ? widen(Br.v[j], (const T *)nullptr) : 0.0f;
                    const float Cn = nv ? widen(Cr.v[j], (const T *)nullptr) : 0.0f;
                    float da;
                    if (S4D) { da = pw; pw *= p1; }
                    else da = fast_exp2(dl * a2[j]);
                    hs[j] = fmaf(da, hs[j], du * Bn);
                    acc = fmaf(hs[j], Cn, acc);
                }
#pragma unroll
                for (int m = 1; m < LPC; m <<= 1) acc += __shfl_xor(acc, m, kWave);
                if (GATE == 1) acc *= widen(rg[s], (const T *)nullptr);
                if (GATE == 2) acc *= silu(widen(rg[s], (const T *)nullptr));
                if (live && g == 0) Store<T>::st(y + (row0 + t) * di + dd, acc);
            }
        }
        if (tb + kSeqBlock < Tlen) {
            publish(buf ^ 1);
#pragma unroll
            for (int s = 0; s < kSeqBlock; s++) { rd[s] = nd[s]; ru[s] = nu[s]; rg[s] = ng[s]; }
        }
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
                           const float *D, const T *gate, int64_t gate_stride, int batch, int Tlen, int di, int ds) {
    constexpr int CPW = kWave / LPC;
    const int tiles = (di + CPW - 1) / CPW;
    const dim3 grid((unsigned)(batch * tiles)), block(kWave);
#define MRS_LAUNCH(G)                                                                              \
    hipLaunchKernelGGL((ssm_scan_seq_kernel<T, LPC, S4D, G>), grid, block, 0, st, h, y, delta, u, Bm, \
                       Cm, bc_stride, a_neg, D, gate, gate_stride, Tlen, di, ds, tiles)
    if (gate_mode == 0) MRS_LAUNCH(0);
    else if (gate_mode == 1) MRS_LAUNCH(1);
    else MRS_LAUNCH(2);
#undef MRS_LAUNCH
    return check_launch("ssm_scan_seq_kernel");
}

template <typename T>
static int launch_seq(hipStream_t st, bool s4d, int gate_mode, float *h, void *y, const void *delta,
                      const void *u, const void *Bm, const void *Cm, int64_t bc_stride,
                      const float *a_neg, const float *D, const void *gate, int64_t gate_stride, int batch, int Tlen,
                      int di, int ds) {
#define MRS_ARGS                                                                                     \
    st, gate_mode, h, (T *)y, (const T *)delta, (const T *)u, (const T *)Bm, (const T *)Cm, bc_stride, \
        a_neg, D, (const T *)gate, gate_stride, batch, Tlen, di, ds
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
// states of a channel in that lane's registers.
//   pass A  chunk_state_kernel: chunk-end state S_c reached from a zero entering
//           state (chunk 0: from the caller's h) and sum_t delta over the chunk,
//           for chunks 0..C-2; saves a copy of the caller's h.
//   pass B  chunk_out_kernel: folds the summaries of the chunks before it into its
//           entering state  h_in(c) = exp(a * sum delta_{c-1}) h_in(c-1) + S_{c-1},
//           then runs the recurrence over its chunk writing y; the last chunk
//           writes the final state back to h.
// The composition law (a,b)o(a',b') = (aa', a'b + b') makes this equal to the
// serial scan up to rounding.
//
// How the B_t / C_t rows (wave-uniform, 16 values each) reach the arithmetic: a wave copies the rows of 16 steps at a
// time into its own 4 KB of LDS as f32 (lane l brings elements 4(l%4)..+3 of row l/4), two such spans ahead of their
// use.  The two consumers read them back in two ways:
//   * the rank-1 state update of pass B runs on the matrix core: every lane reads 16 bytes, lane l gets X[4(l%4) + k] in
//     register k, and v_mfma_f32_4x4x1 number k with register k as its A operand gives result register a of lane l
//     A(lane 4(l/4)+a) * B(lane l) = X[4a+k] * (delta u)[l]  --  so state n = 4a+k lives in state register 4k+a (a 4x4
//     transpose of the natural order, kStateOfReg below);
//   * the multiply-adds with a row as the uniform factor (the output dot of pass B, the summary of pass A) take the
//     row as ordinary registers: four 16-byte LDS reads with one address for all lanes put the whole row on every
//     lane.  A SIMD issues two plain f32 instructions per issue slot when two of its waves have one ready, but an
//     instruction with a DPP operand (the quad broadcast these kernels used before) takes the slot alone: sixteen of
//     them per step cost sixteen slots, sixteen plain ones and the four reads cost ten.
// ---------------------------------------------------------------------------
struct SplitPlan {
    int nchunk;  // C
    int len;     // L
};

constexpr int kGroup = 8;            // steps per activation prefetch group
constexpr int kSpan = 2 * kGroup;    // steps per loop iteration and per staged block of B / C rows; chunk lengths are multiples

// Chunk count: the waves of a launch (chunks x batch rows x channel tiles) should come to about three per SIMD -- what
// keeps the vector ALU issuing -- and fill the 1024 SIMDs of the chip evenly: a SIMD with one wave more than the others
// sets the time of the launch (4 x 4096 x 5120: 9 chunks = 2880 waves 375 us, 10 chunks = 3200 waves 404 us).
constexpr int kSimds = 1024;   // 256 compute units x 4
static SplitPlan make_split_plan(int batch, int Tlen, int di) {
    const int tiles = (di + kWave - 1) / kWave;
    const int64_t base = (int64_t)batch * tiles;
    static const int target = [] { const char *e = getenv("MRS_SCAN_TARGET_WAVES"); return e ? atoi(e) : 0; }();
    int cmax = 32;                               // the entering-state fold is O(C) per wave
    if (cmax > Tlen / 32) cmax = Tlen / 32;      // chunks of at least 32 steps
    int c;
    if (target > 0) {
        c = (int)((target + base - 1) / base);
    } else {
        // between two and three and a half waves per SIMD, the fullest last round wins; on a tie three waves per SIMD
        // (they hide each other's waits: 4 x 4096 x 5120 takes 350 us with 2880 waves, 367 us with 1920, 400 us with
        // 3840), else fewer waves
        int lo = (int)(2 * kSimds / base), hi = (int)((7 * kSimds / 2 + base - 1) / base);
        if (lo < 2) lo = 2;
        if (hi < lo) hi = lo;
        c = hi;
        double best = -1.0;
        bool best3 = false;
        for (int k = lo; k <= hi; k++) {
            const int64_t waves = k * base, rounds = (waves + kSimds - 1) / kSimds;
            const double fill = (double)waves / (double)(rounds * kSimds);
            if (fill > best + 1e-9 || (fill > best - 1e-9 && rounds == 3 && !best3)) { best = fill; c = k; best3 = rounds == 3; }
        }
    }
    if (c > cmax) c = cmax;
    if (c < 1) c = 1;
    int len = (Tlen + c - 1) / c;
    len = (len + kSpan - 1) / kSpan * kSpan;
    c = (Tlen + len - 1) / len;
    return {c, len};
}

struct SplitWs {
    unsigned *flags;  // [B][tiles][kMaxChunks]: chunk summary published (the one-launch route)
    unsigned *done;   // [B][tiles]: waves that have folded their entering state
    size_t flag_words;
    float *h0copy;  // [B][16][di]
    float *S;       // [B][C-1][16][di]
    float *sumd;    // [B][C-1][di]
    size_t floats;  // whole workspace, in 4-byte words
};

constexpr int kMaxChunks = 32;

// The flag area comes first and has one size whatever the shape of the call, so that a buffer shared by calls of
// different shapes (the library's static one, an engine's scratch) never has one call's summaries where another call's
// flags are: it stays all zero between calls.  A call with more (batch row, channel tile) pairs than it holds takes the
// two-launch form.
constexpr size_t kFlagAreaWords = 65536;   // 256 KB: 1985 pairs of kMaxChunks flags + a counter
static bool flags_fit(int batch, int di) {
    return (size_t)batch * (size_t)((di + kWave - 1) / kWave) * (kMaxChunks + 1) <= kFlagAreaWords;
}
static SplitWs carve_workspace(float *base, int batch, int Tlen, int di, int nchunk) {
    (void)Tlen;
    SplitWs w;
    const size_t tiles = (size_t)((di + kWave - 1) / kWave);
    w.flags = reinterpret_cast<unsigned *>(base);
    w.done = w.flags + (size_t)batch * tiles * kMaxChunks;
    w.flag_words = kFlagAreaWords;
    size_t o = kFlagAreaWords;
    w.h0copy = base + o; o += (size_t)batch * 16 * di;
    w.S = base + o; o += (size_t)batch * (nchunk - 1) * 16 * di;
    w.sumd = base + o; o += (size_t)batch * (nchunk - 1) * di;
    w.floats = o;
    return w;
}

// Per-lane activation access through a buffer resource: address = base (scalar
// registers) + per-step scalar offset + per-lane 32-bit offset, so the row walk costs
// no vector ALU work.  num_records bounds the slab; offsets here stay below 2^31.
template <typename T> struct LaneBuf {
    __amdgpu_buffer_rsrc_t r;
    __device__ __forceinline__ LaneBuf(const T *base, int64_t elems) {
        r = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(base), 0, (int)(elems * (int64_t)sizeof(T)), 0x00020000);
    }
    __device__ __forceinline__ typename RawElem<T>::type ld(unsigned voff, unsigned soff) const {
        if constexpr (sizeof(T) == 4) return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
        else return __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0);
    }
    __device__ __forceinline__ void st(float v, unsigned voff, unsigned soff) const {
        if constexpr (sizeof(T) == 4) {
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, voff, soff, 0);
        } else {
            const T t = (T)v;
            __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(uint16_t, t), r, voff, soff, 0);
        }
    }
};

typedef float v4f __attribute__((ext_vector_type(4)));

// Raw activation values of the T-split kernels sit zero-extended in a register of their own: as 16-bit values the
// compiler packs them in pairs and spends vector instructions on packing and unpacking.
template <typename T> struct Raw32 { using type = uint32_t; };
template <> struct Raw32<float> { using type = float; };
__device__ __forceinline__ float widen32(float v, const float *) { return v; }
__device__ __forceinline__ float widen32(uint32_t v, const bf16_t *) { return __uint_as_float(v << 16); }
__device__ __forceinline__ float widen32(uint32_t v, const f16_t *) { return (float)__builtin_bit_cast(_Float16, (uint16_t)v); }

// state held in state register r (see the header comment): a 4x4 transpose, its own inverse
__host__ __device__ constexpr int kStateOfReg(int r) { return 4 * (r % 4) + r / 4; }

// A lane's piece of a span of rows: elements 4(l%4)..+3 of row l/4, raw (two dwords of 16-bit values or four floats).
template <typename T> struct RowPiece { uint32_t w[sizeof(T) == 4 ? 4 : 2]; };
template <typename T>
__device__ __forceinline__ void piece_ld(RowPiece<T> &o, const T *rows, int64_t stride, int row) {
    const uint32_t *p = reinterpret_cast<const uint32_t *>(rows + (int64_t)row * stride + 4 * (threadIdx.x & 3));
#pragma unroll
    for (int j = 0; j < (int)(sizeof(T) == 4 ? 4 : 2); j++) o.w[j] = p[j];
}
__device__ __forceinline__ v4f piece_widen(const RowPiece<float> &r, const float *) {
    return v4f{__uint_as_float(r.w[0]), __uint_as_float(r.w[1]), __uint_as_float(r.w[2]), __uint_as_float(r.w[3])};
}
__device__ __forceinline__ v4f piece_widen(const RowPiece<bf16_t> &r, const bf16_t *) {
    return v4f{__uint_as_float(r.w[0] << 16), __uint_as_float(r.w[0] & 0xffff0000u), __uint_as_float(r.w[1] << 16),
               __uint_as_float(r.w[1] & 0xffff0000u)};
}
__device__ __forceinline__ v4f piece_widen(const RowPiece<f16_t> &r, const f16_t *) {
    return v4f{(float)__builtin_bit_cast(_Float16, (uint16_t)(r.w[0] & 0xffffu)), (float)__builtin_bit_cast(_Float16, (uint16_t)(r.w[0] >> 16)),
               (float)__builtin_bit_cast(_Float16, (uint16_t)(r.w[1] & 0xffffu)), (float)__builtin_bit_cast(_Float16, (uint16_t)(r.w[1] >> 16))};
}

// The wave's staged rows: [slot = span parity][row][16] f32, one such array per tensor.
struct StagedRows {
    float v[2][kSpan][16];
    __device__ __forceinline__ void publish(int slot, const v4f &x) {
        *reinterpret_cast<v4f *>(&v[slot][threadIdx.x >> 2][4 * (threadIdx.x & 3)]) = x;
    }
    __device__ __forceinline__ v4f read(int slot, int row) const {
        return *reinterpret_cast<const v4f *>(&v[slot][row][4 * (threadIdx.x & 3)]);
    }
    // elements 4q..4q+3 of a row, the same on every lane
    __device__ __forceinline__ v4f read_all(int slot, int row, int q) const {
        return *reinterpret_cast<const v4f *>(&v[slot][row][4 * q]);
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

// The same with the power chain as a tree (depth 4 instead of 15), 15 multiplies all the same.
template <bool S4D>
__device__ __forceinline__ void decay16_tree(float dl, const float (&a2)[16], float (&da)[16]) {
    if (S4D) {
        const float p = fast_exp2(dl * a2[0]);
        da[0] = p; da[1] = p * p; da[2] = da[1] * p; da[3] = da[1] * da[1];
#pragma unroll
        for (int j = 4; j < 8; j++) da[j] = da[3] * da[j - 4];
#pragma unroll
        for (int j = 8; j < 16; j++) da[j] = da[7] * da[j - 8];
    } else {
#pragma unroll
        for (int j = 0; j < 16; j++) da[j] = fast_exp2(dl * a2[j]);
    }
}

template <bool S4D>
__device__ __forceinline__ void load_a2(float (&a2)[16], const float *__restrict__ a_neg, int d) {
#pragma unroll
    for (int j = 0; j < 16; j++) a2[j] = a_neg[(int64_t)d * 16 + j] * kLog2e;
    if (S4D) {
#pragma unroll
        for (int j = 1; j < 16; j++) a2[j] = a2[0] * (float)(j + 1);
    }
}

// Entering state of chunk c (c >= 1) from the summaries of chunks 0..c-1, in direct form:
//   h_in(c) = sum_{k<c} exp(a * sum_{k<m<c} sumdelta_m) (.) S_k        (S_0 already holds h0's share)
// The terms are independent; the summaries are fetched four chunks at a time (68 loads in flight), so the fold costs
// a few memory round trips instead of one per chunk -- every wave of pass B sits through it before its first step.
// hs[n] is state n.
constexpr int kFoldBatch = 4;
// A float another wave of the same launch has published (the one-launch route): a relaxed load at agent scope, so that it
// is served from where that wave's relaxed agent-scope store put it, whichever part of the chip either wave runs on.
// Between launches the plain load does (the kernel boundary publishes).
template <bool FUSED> __device__ __forceinline__ float pub_ld(const float *p) {
    if constexpr (FUSED) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else return *p;
}
template <bool FUSED> __device__ __forceinline__ void pub_st(float *p, float v) {
    if constexpr (FUSED) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}

template <bool S4D, bool FUSED = false>
__device__ __forceinline__ void fold_entering_state(float (&hs)[16], const float (&a2)[16],
                                                    const float *__restrict__ S, const float *__restrict__ sumd,
                                                    int b, int c, int nchunk, int di, int dd) {
    const int64_t sbase = (int64_t)b * (nchunk - 1);
#pragma unroll
    for (int j = 0; j < 16; j++) hs[j] = pub_ld<FUSED>(S + ((sbase + c - 1) * 16 + j) * di + dd);  // k = c-1: weight 1
    float suffix = 0.0f;  // sum of sumdelta_m over k < m < c
    for (int k0 = c - 2; k0 >= 0; k0 -= kFoldBatch) {
        float Sv[kFoldBatch][16], sm[kFoldBatch];
#pragma unroll
        for (int i = 0; i < kFoldBatch; i++) {
            const int k = max(k0 - i, 0);     // past the front: chunk 0 again, loaded and not used
            sm[i] = pub_ld<FUSED>(sumd + (sbase + k + 1) * di + dd);
#pragma unroll
            for (int j = 0; j < 16; j++) Sv[i][j] = pub_ld<FUSED>(S + ((sbase + k) * 16 + j) * di + dd);
        }
#pragma unroll
        for (int i = 0; i < kFoldBatch; i++) {
            if (k0 - i >= 0) {                // wave-uniform
                suffix += sm[i];
                float da[16];
                decay16_tree<S4D>(suffix, a2, da);
#pragma unroll
                for (int j = 0; j < 16; j++) hs[j] = fmaf(da[j], Sv[i][j], hs[j]);
            }
        }
    }
}

// Issue priority by progress.  The instruction arbiter of a SIMD serves its oldest ready wave first, so waves that start
// together finish one after the other and the last one ends up alone on the SIMD, where it cannot fill the vector ALU
// (measured: three waves per SIMD finished at 73, 103 and 132 thousand ticks).  A wave therefore lowers its own priority
// as it gets through its chunk -- after 1/2, 3/4 and 7/8 of its spans -- so whoever is behind is served first and the
// waves of a SIMD stay together until the last eighth.
__device__ __forceinline__ void set_progress_priority(int done, int total) {
    if (done * 8 >= total * 7) __builtin_amdgcn_s_setprio(0);
    else if (done * 4 >= total * 3) __builtin_amdgcn_s_setprio(1);
    else if (done * 2 >= total) __builtin_amdgcn_s_setprio(2);
    else __builtin_amdgcn_s_setprio(3);
}

// Lanes of a partial channel tile beyond d_inner address their activations at an offset outside every buffer
// resource: their loads return zero and their stores are dropped, so the time loops carry no lane predicate.
constexpr unsigned kDeadLaneOffset = 0x7f000000u;

// Pass A for the wave (batch row b, chunk c < nchunk - 1, channel tile).  Chunk lengths are multiples of kSpan: every
// step of the chunk exists, so the walk has no tail.  FUSED: the wave is part of the one-launch route -- the summary is
// published to the other waves of the launch (relaxed agent-scope stores, then the chunk's flag), and chunk 0 hands
// the caller's state back in h_keep instead of through the h0copy buffer.
template <typename T, bool S4D, bool FUSED>
__device__ __forceinline__ void pass_a_body(
    StagedRows &Bs, const float *__restrict__ h, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, int64_t bc_stride,
    const float *__restrict__ a_neg, float *__restrict__ h0copy, float *__restrict__ S,
    float *__restrict__ sumd, unsigned *__restrict__ flags, float (&h_keep)[16],
    int Tlen, int di, int tiles, int nchunk, int len, int b, int c, int tile) {
    using raw_t = typename Raw32<T>::type;
    const int nc1 = nchunk - 1;
    const int d0 = tile * kWave;
    const bool live = d0 + (int)threadIdx.x < di;
    const int dd = live ? d0 + (int)threadIdx.x : di - 1;   // plain loads of dead lanes shadow the last live channel
    const unsigned lxb = live ? threadIdx.x * (unsigned)sizeof(T) : kDeadLaneOffset;

    float hs[16], a2[16];   // hs[n]: state n
    load_a2<S4D>(a2, a_neg, dd);
#pragma unroll
    for (int j = 0; j < 16; j++) hs[j] = 0.0f;
    auto load_entering = [&]() {   // chunk 0 alone starts from the caller's state
        if (c == 0) {
#pragma unroll
            for (int j = 0; j < 16; j++) {
                hs[j] = h[((int64_t)b * di + dd) * 16 + j];
                if constexpr (FUSED) h_keep[j] = hs[j];
                else if (live) h0copy[((int64_t)b * 16 + j) * di + dd] = hs[j];
            }
        }
    };
    if (!S4D) load_entering();   // the forward walk needs it at once
    const int t0 = c * len;
    const int64_t row0 = (int64_t)b * Tlen;
    const int64_t slab = (int64_t)Tlen * di - d0;  // elements from this wave's base to the end of batch row b
    const LaneBuf<T> dbuf(delta + row0 * di + d0, slab), ubuf(u + row0 * di + d0, slab);
    const unsigned row_bytes = (unsigned)di * (unsigned)sizeof(T);
    const T *Bp = Bm + row0 * bc_stride;
    float sd = 0.0f;
    const int nspans = len / kSpan;
    const int prow = threadIdx.x >> 2;   // the row of a span this lane stages

    raw_t rdA[kGroup], ruA[kGroup], rdB[kGroup], ruB[kGroup];
    auto load_group = [&](raw_t (&rd)[kGroup], raw_t (&ru)[kGroup], int tg) {   // steps tg .. tg+7 (tg clamped into the chunk)
        unsigned o = (unsigned)max(tg, t0) * row_bytes;
#pragma unroll
        for (int k = 0; k < kGroup; k++, o += row_bytes) {
            rd[k] = dbuf.ld(lxb, o);
            ru[k] = ubuf.ld(lxb, o);
        }
    };
    RowPiece<T> nb;
    if (S4D) {
        // Direct form, walking the chunk backwards: the weight of step s in the chunk-end
        // state is prod_{r>s} exp(delta_r a_n) = x_s^(n+1) with x_s = 2^(a2[0] * sum_{r>s} delta_r),
        // so one exp, a power chain and one multiply-add per state -- no decay of a running state.
        float S16[16];   // S16[n]: state n
#pragma unroll
        for (int j = 0; j < 16; j++) S16[j] = 0.0f;
        // spans are walked last to first; span s sits in slot s & 1, span s-1 is published while s is computed and
        // the rows of span s-2 requested
        // everything the first steps need is requested before any of it is used (loads come back in the order they were
        // issued): the rows of the last span, those of the span before it, the first group of steps, and -- chunk 0 --
        // the entering state, which the backward walk needs only at its end.  One after the other they were three memory
        // round trips in front of the first step, for every wave of the launch at the same time.
        {
            RowPiece<T> first;
            piece_ld(first, Bp, bc_stride, t0 + (nspans - 1) * kSpan + prow);
            piece_ld(nb, Bp, bc_stride, t0 + max(nspans - 2, 0) * kSpan + prow);
            load_group(rdB, ruB, t0 + (nspans - 1) * kSpan + kGroup);
            load_entering();
            Bs.publish((nspans - 1) & 1, piece_widen(first, (const T *)nullptr));
        }
        for (int sp = nspans - 1; sp >= 0; sp--) {
            const int ts = t0 + sp * kSpan, slot = sp & 1;
            set_progress_priority(nspans - 1 - sp, nspans);
            Bs.publish(slot ^ 1, piece_widen(nb, (const T *)nullptr));
            piece_ld(nb, Bp, bc_stride, t0 + max(sp - 2, 0) * kSpan + prow);
            load_group(rdA, ruA, ts);
            auto back = [&](const raw_t (&rd)[kGroup], const raw_t (&ru)[kGroup], int base) {
#pragma unroll
                for (int k = kGroup - 1; k >= 0; k--) {
                    const int j = base + k;                               // row of the span
                    v4f ball[4];
#pragma unroll
                    for (int q = 0; q < 4; q++) ball[q] = Bs.read_all(slot, j, q);
                    const float dl = widen32(rd[k], (const T *)nullptr);
                    const float uu = widen32(ru[k], (const T *)nullptr);
                    const float x = fast_exp2(a2[0] * sd);
                    float v = x * (dl * uu);
                    sd += dl;
#pragma unroll
                    for (int n = 0; n < 16; n++) {
                        S16[n] = fmaf(v, ball[n >> 2][n & 3], S16[n]);
                        if (n < 15) v *= x;
                    }
                }
            };
            back(rdB, ruB, kGroup);
            load_group(rdB, ruB, ts - kGroup);
            back(rdA, ruA, 0);
        }
        // entering state (chunk 0 only; zero otherwise) decayed over the whole chunk
        float da[16];
        decay16<true>(sd, a2, da);
#pragma unroll
        for (int j = 0; j < 16; j++) hs[j] = fmaf(da[j], hs[j], S16[j]);
    } else {
        // General A: the recurrence itself, forwards, with the rank-1 update on the matrix core as in pass B.
        float hr[16];   // hr[r]: state kStateOfReg(r)
#pragma unroll
        for (int r = 0; r < 16; r++) hr[r] = hs[kStateOfReg(r)];
        {
            RowPiece<T> first;   // requested together, as in the backward walk above
            piece_ld(first, Bp, bc_stride, t0 + prow);
            piece_ld(nb, Bp, bc_stride, t0 + min(1, nspans - 1) * kSpan + prow);
            load_group(rdA, ruA, t0);
            Bs.publish(0, piece_widen(first, (const T *)nullptr));
        }
        v4f bv = Bs.read(0, 0);
        for (int sp = 0; sp < nspans; sp++) {
            const int ts = t0 + sp * kSpan, slot = sp & 1;
            set_progress_priority(sp, nspans);
            Bs.publish(slot ^ 1, piece_widen(nb, (const T *)nullptr));
            piece_ld(nb, Bp, bc_stride, t0 + min(sp + 2, nspans - 1) * kSpan + prow);
            load_group(rdB, ruB, ts + kGroup);
            auto fwd = [&](const raw_t (&rd)[kGroup], const raw_t (&ru)[kGroup], int base) {
#pragma unroll
                for (int k = 0; k < kGroup; k++) {
                    const int j = base + k;
                    const v4f bcur = bv;
                    bv = j < kSpan - 1 ? Bs.read(slot, j + 1) : Bs.read(slot ^ 1, 0);
                    const float dl = widen32(rd[k], (const T *)nullptr);
                    const float uu = widen32(ru[k], (const T *)nullptr);
                    const float du = dl * uu;
                    float da[16];
                    decay16_tree<false>(dl, a2, da);
                    sd += dl;
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        v4f hq = {hr[4 * q] * da[kStateOfReg(4 * q)], hr[4 * q + 1] * da[kStateOfReg(4 * q + 1)],
                                  hr[4 * q + 2] * da[kStateOfReg(4 * q + 2)], hr[4 * q + 3] * da[kStateOfReg(4 * q + 3)]};
                        hq = __builtin_amdgcn_mfma_f32_4x4x1f32(bcur[q], du, hq, 0, 0, 0);
#pragma unroll
                        for (int i = 0; i < 4; i++) hr[4 * q + i] = hq[i];
                    }
                }
            };
            fwd(rdA, ruA, 0);
            load_group(rdA, ruA, min(ts + kSpan, t0 + len - kGroup));
            fwd(rdB, ruB, kGroup);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) hs[kStateOfReg(r)] = hr[r];
    }
    if (live) {
        const int64_t sbase = (int64_t)b * nc1 + c;
#pragma unroll
        for (int j = 0; j < 16; j++) pub_st<FUSED>(S + (sbase * 16 + j) * di + dd, hs[j]);
        pub_st<FUSED>(sumd + sbase * di + dd, sd);
    }
    if constexpr (FUSED) {
        // the summary has arrived where the other waves will look for it before the flag says so
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (threadIdx.x == 0)
            __hip_atomic_store(flags + ((int64_t)b * tiles + tile) * kMaxChunks + c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <typename T, bool S4D>
__global__ __launch_bounds__(kWave) void chunk_state_kernel(
    const float *__restrict__ h, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, int64_t bc_stride,
    const float *__restrict__ a_neg, float *__restrict__ h0copy, float *__restrict__ S,
    float *__restrict__ sumd, int Tlen, int di, int tiles, int nchunk, int len) {
    __shared__ alignas(16) StagedRows Bs;
    const int nc1 = nchunk - 1;   // chunks 0 .. nchunk-2 only
    const int tile = blockIdx.x % tiles;
    const int rest = blockIdx.x / tiles;
    float unused[16];
    pass_a_body<T, S4D, false>(Bs, h, delta, u, Bm, bc_stride, a_neg, h0copy, S, sumd, nullptr, unused, Tlen, di, tiles, nchunk, len,
                               rest / nc1, rest % nc1, tile);
}

// Pass B.  The time loop has no tail and no lane predicate: rows at and beyond T lie outside the buffer resources
// (loads return zero: delta = 0 leaves the state as it is, stores are dropped), and so do the lanes of a partial tile.
// FUSED (the one-launch route): the summaries of the chunks before this one are other waves' work of the same launch --
// the wave waits for their flags (a bounded wait: every wave reaches its end whatever happens), folds them through
// agent-scope loads, and the last wave of a (batch row, channel tile) to have folded clears that pair's flags and
// counter again, so that the flag area is all zero between launches.  Chunk 0 takes its entering state from h_keep.
constexpr int kFlagSpinLimit = 1 << 22;
template <typename T, bool S4D, int GATE, bool FUSED>
__device__ __forceinline__ void pass_b_body(
    StagedRows &Bs, StagedRows &Cs, float *__restrict__ h, T *__restrict__ y, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, const T *__restrict__ Cm, int64_t bc_stride,
    const float *__restrict__ a_neg, const float *__restrict__ Dp, const T *__restrict__ gate, int64_t gate_stride,
    const float *__restrict__ h0copy, const float *__restrict__ S, const float *__restrict__ sumd,
    unsigned *__restrict__ flags, unsigned *__restrict__ done, const float (&h_keep)[16],
    int Tlen, int di, int tiles, int nchunk, int len, int b, int c, int tile) {
    using raw_t = typename Raw32<T>::type;
    const int d0 = tile * kWave;
    const bool live = d0 + (int)threadIdx.x < di;
    const int dd = live ? d0 + (int)threadIdx.x : di - 1;
    const unsigned lxb = live ? threadIdx.x * (unsigned)sizeof(T) : kDeadLaneOffset;

    const int t0 = c * len, t1 = min(Tlen, t0 + len);
    const int tl = Tlen - 1;
    const int64_t row0 = (int64_t)b * Tlen;
    const int64_t slab = (int64_t)Tlen * di - d0;
    const LaneBuf<T> dbuf(delta + row0 * di + d0, slab), ubuf(u + row0 * di + d0, slab);
    const LaneBuf<T> gbuf(GATE ? gate + row0 * gate_stride + d0 : delta, GATE ? (int64_t)Tlen * gate_stride - d0 : 0), ybuf(y + row0 * di + d0, slab);
    const unsigned row_bytes = (unsigned)di * (unsigned)sizeof(T);
    const unsigned gate_row_bytes = (unsigned)gate_stride * (unsigned)sizeof(T);
    const T *Bp = Bm + row0 * bc_stride, *Cp = Cm + row0 * bc_stride;
    const int prow = threadIdx.x >> 2;

    raw_t rdA[kGroup], ruA[kGroup], rgA[kGroup], rdB[kGroup], ruB[kGroup], rgB[kGroup];
    auto load_group = [&](raw_t (&rd)[kGroup], raw_t (&ru)[kGroup], raw_t (&rg)[kGroup], int tg) {
        unsigned o = (unsigned)tg * row_bytes, og = (unsigned)tg * gate_row_bytes;
#pragma unroll
        for (int k = 0; k < kGroup; k++, o += row_bytes, og += gate_row_bytes) {
            rd[k] = dbuf.ld(lxb, o);
            ru[k] = ubuf.ld(lxb, o);
            if (GATE) rg[k] = gbuf.ld(lxb, og);
        }
    };
    const int nspans = (t1 - t0 + kSpan - 1) / kSpan;
    // Everything the first steps need is requested before the entering state is folded, so the memory round trips of
    // the prologue overlap instead of following one another (it is a startup bubble for the whole chip: all waves of a
    // launch are in it at the same time).
    RowPiece<T> nb, nc, fb, fc;
    piece_ld(fb, Bp, bc_stride, min(t0 + prow, tl));
    piece_ld(fc, Cp, bc_stride, min(t0 + prow, tl));
    piece_ld(nb, Bp, bc_stride, min(t0 + kSpan + prow, tl));
    piece_ld(nc, Cp, bc_stride, min(t0 + kSpan + prow, tl));
    load_group(rdA, ruA, rgA, t0);
    const float Dd = Dp[dd];

    float hn[16], a2[16], hs[16], ar[16];   // hn[n]: state n; hs[r], ar[r]: state kStateOfReg(r)
    bool poison = false;
    load_a2<S4D>(a2, a_neg, dd);
    if (c == 0) {
#pragma unroll
        for (int j = 0; j < 16; j++) hn[j] = FUSED ? h_keep[j] : h0copy[((int64_t)b * 16 + j) * di + dd];
    } else {
        if constexpr (FUSED) {
            unsigned *fl = flags + ((int64_t)b * tiles + tile) * kMaxChunks;
            bool arrived = false;
            for (int spin = 0; spin < kFlagSpinLimit && !arrived; spin++) {
                const unsigned f = (int)threadIdx.x < c ? __hip_atomic_load(fl + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 1u;
                arrived = __builtin_amdgcn_ballot_w64(f == 0u) == 0;
                if (!arrived) __builtin_amdgcn_s_sleep(8);
            }
            asm volatile("" ::: "memory");
            // a summary that never came (seconds of waiting: the flag area was not zero, or two calls share the buffer):
            // the wave goes on to its end, and its outputs say so -- NaN, not a plausible number
            poison = !arrived;
        }
        fold_entering_state<S4D, FUSED>(hn, a2, S, sumd, b, c, nchunk, di, dd);
        if constexpr (FUSED) {
            if (poison) {
#pragma unroll
                for (int j = 0; j < 16; j++) hn[j] = __builtin_nanf("");
            }
            // every summary is in registers (the fold consumed them); the last of the nchunk - 1 folding waves of this
            // (batch row, channel tile) leaves the pair's flags and counter zero for the next launch
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            unsigned *fl = flags + ((int64_t)b * tiles + tile) * kMaxChunks;
            unsigned *dn = done + (int64_t)b * tiles + tile;
            unsigned old = 0;
            if (threadIdx.x == 0) old = __hip_atomic_fetch_add(dn, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            old = __builtin_amdgcn_readfirstlane(old);
            if (old == (unsigned)(nchunk - 2)) {
                if ((int)threadIdx.x < nchunk - 1) __hip_atomic_store(fl + threadIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (threadIdx.x == 0) __hip_atomic_store(dn, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 16; r++) { hs[r] = hn[kStateOfReg(r)]; ar[r] = a2[kStateOfReg(r)]; }
    Bs.publish(0, piece_widen(fb, (const T *)nullptr));
    Cs.publish(0, piece_widen(fc, (const T *)nullptr));
    v4f bv = Bs.read(0, 0);
    for (int sp = 0; sp < nspans; sp++) {
        const int ts = t0 + sp * kSpan, slot = sp & 1;
        set_progress_priority(sp, nspans);
        // span sp+1 into the other slot (its rows were requested a span ago), then the request for span sp+2
        Bs.publish(slot ^ 1, piece_widen(nb, (const T *)nullptr));
        Cs.publish(slot ^ 1, piece_widen(nc, (const T *)nullptr));
        piece_ld(nb, Bp, bc_stride, min(ts + 2 * kSpan + prow, tl));
        piece_ld(nc, Cp, bc_stride, min(ts + 2 * kSpan + prow, tl));
        load_group(rdB, ruB, rgB, ts + kGroup);
        auto steps = [&](const raw_t (&rd)[kGroup], const raw_t (&ru)[kGroup], const raw_t (&rg)[kGroup], int base) {
            unsigned yo = (unsigned)(ts + base) * row_bytes;
#pragma unroll
            for (int k = 0; k < kGroup; k++, yo += row_bytes) {
                const int j = base + k;
                const v4f bcur = bv;
                bv = j < kSpan - 1 ? Bs.read(slot, j + 1) : Bs.read(slot ^ 1, 0);   // the B row of the next step, a quad piece per lane
                v4f call[4];
#pragma unroll
                for (int q = 0; q < 4; q++) call[q] = Cs.read_all(slot, j, q);      // this step's C row, whole, on every lane
                const float dl = widen32(rd[k], (const T *)nullptr);
                const float uu = widen32(ru[k], (const T *)nullptr);
                const float du = dl * uu;
                float da[16];
                if (S4D) {
                    float dn[16];
                    decay16_tree<true>(dl, a2, dn);
#pragma unroll
                    for (int r = 0; r < 16; r++) da[r] = dn[kStateOfReg(r)];
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r++) da[r] = fast_exp2(dl * ar[r]);
                }
                v4f hq[4];
#pragma unroll
                for (int q = 0; q < 4; q++)
                    hq[q] = v4f{hs[4 * q] * da[4 * q], hs[4 * q + 1] * da[4 * q + 1], hs[4 * q + 2] * da[4 * q + 2], hs[4 * q + 3] * da[4 * q + 3]};
                // the four matrix instructions back to back: one between vector instructions costs a pipeline switch each way
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int q = 0; q < 4; q++) hq[q] = __builtin_amdgcn_mfma_f32_4x4x1f32(bcur[q], du, hq[q], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int i = 0; i < 4; i++) hs[4 * q + i] = hq[q][i];
                float acc, e;
                const float z = GATE ? widen32(rg[k], (const T *)nullptr) : 0.0f;
                acc = Dd * uu;
                e = fast_exp2(z * -kLog2e);
#pragma unroll
                for (int r = 0; r < 16; r++) acc = fmaf(call[kStateOfReg(r) >> 2][kStateOfReg(r) & 3], hs[r], acc);
                if (GATE == 1) acc *= z;
                if (GATE == 2) acc *= z * fast_rcp(1.0f + e);
                ybuf.st(acc, lxb, yo);
            }
        };
        steps(rdA, ruA, rgA, 0);
        load_group(rdA, ruA, rgA, ts + kSpan);
        steps(rdB, ruB, rgB, kGroup);
    }
    if (c == nchunk - 1 && live) {
#pragma unroll
        for (int r = 0; r < 16; r++) h[((int64_t)b * di + dd) * 16 + kStateOfReg(r)] = hs[r];
    }
}

template <typename T, bool S4D, int GATE>
__global__ __launch_bounds__(kWave) void chunk_out_kernel(
    float *__restrict__ h, T *__restrict__ y, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, const T *__restrict__ Cm, int64_t bc_stride,
    const float *__restrict__ a_neg, const float *__restrict__ Dp, const T *__restrict__ gate, int64_t gate_stride,
    const float *__restrict__ h0copy, const float *__restrict__ S, const float *__restrict__ sumd,
    int Tlen, int di, int tiles, int nchunk, int len) {
    __shared__ alignas(16) StagedRows Bs, Cs;
    const int tile = blockIdx.x % tiles;
    const int rest = blockIdx.x / tiles;
    const float unused[16] = {};
    pass_b_body<T, S4D, GATE, false>(Bs, Cs, h, y, delta, u, Bm, Cm, bc_stride, a_neg, Dp, gate, gate_stride, h0copy, S, sumd, nullptr,
                                     nullptr, unused, Tlen, di, tiles, nchunk, len, rest / nchunk, rest % nchunk, tile);
}

// Both passes in one launch: the wave (chunk c, batch row b, channel tile) summarises its chunk, publishes the summary,
// waits for the chunks before it and walks its chunk again for the outputs.  Workgroups are numbered chunk-major, so a
// wave only ever waits for waves with smaller indices (dispatched before it); the last chunk has nothing to summarise
// and goes straight to waiting.  The flag area (kMaxChunks flags and a counter per (batch row, channel tile)) must be all
// zero when the launch starts and is all zero again when it ends.
template <typename T, bool S4D, int GATE>
__global__ __launch_bounds__(kWave) void scan_fused_kernel(
    float *__restrict__ h, T *__restrict__ y, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bm, const T *__restrict__ Cm, int64_t bc_stride,
    const float *__restrict__ a_neg, const float *__restrict__ Dp, const T *__restrict__ gate, int64_t gate_stride,
    float *__restrict__ S, float *__restrict__ sumd, unsigned *__restrict__ flags, unsigned *__restrict__ done,
    int batch, int Tlen, int di, int tiles, int nchunk, int len) {
    __shared__ alignas(16) StagedRows Bs, Cs;
    const int tile = blockIdx.x % tiles;
    const int rest = blockIdx.x / tiles;
    const int b = rest % batch, c = rest / batch;
    float h_keep[16];
#pragma unroll
    for (int j = 0; j < 16; j++) h_keep[j] = 0.0f;
    if (c < nchunk - 1)
        pass_a_body<T, S4D, true>(Bs, h, delta, u, Bm, bc_stride, a_neg, nullptr, S, sumd, flags, h_keep, Tlen, di, tiles, nchunk, len, b, c, tile);
    pass_b_body<T, S4D, GATE, true>(Bs, Cs, h, y, delta, u, Bm, Cm, bc_stride, a_neg, Dp, gate, gate_stride, nullptr, S, sumd, flags, done,
                                    h_keep, Tlen, di, tiles, nchunk, len, b, c, tile);
}

// clears the flag area of the one-launch route (a kernel, not a memset: the call may be under stream capture)
__global__ __launch_bounds__(256) void scan_flags_clear_kernel(unsigned *__restrict__ p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

template <typename T> struct IsF32 { static constexpr bool value = false; };
template <> struct IsF32<float> { static constexpr bool value = true; };

// one_launch: 0 = two launches (pass A, pass B); 1 = one launch behind a small kernel that clears the flag area;
// 2 = one launch, the caller vouches that the flag area is all zero (MRS_SCAN_FLAGS_ZERO, or the library's own buffer)
template <typename T, bool S4D>
static int launch_split_s4d(hipStream_t st, int gate_mode, float *h, T *y, const T *delta, const T *u,
                            const T *Bm, const T *Cm, int64_t bc_stride, const float *a_neg,
                            const float *D, const T *gate, int64_t gate_stride, float *ws, SplitPlan plan, int batch,
                            int Tlen, int di, int one_launch) {
    const int tiles = (di + kWave - 1) / kWave;
    const int C = plan.nchunk, L = plan.len;
    const SplitWs w = carve_workspace(ws, batch, Tlen, di, C);
    const dim3 block(kWave);
    const dim3 gridA((unsigned)(batch * (C - 1) * tiles)), gridB((unsigned)(batch * C * tiles));
    if (one_launch) {
        if (one_launch == 1) {
            const int used = batch * tiles * (kMaxChunks + 1);   // the words this shape's waves touch
            hipLaunchKernelGGL(scan_flags_clear_kernel, dim3((unsigned)((used + 255) / 256)), dim3(256), 0, st, w.flags, used);
            int rc = check_launch("scan_flags_clear_kernel");
            if (rc) return rc;
        }
#define MRS_LAUNCH(G)                                                                                        \
    hipLaunchKernelGGL((scan_fused_kernel<T, S4D, G>), gridB, block, 0, st, h, y, delta, u, Bm, Cm, bc_stride, \
                       a_neg, D, gate, gate_stride, w.S, w.sumd, w.flags, w.done, batch, Tlen, di, tiles, C, L)
        if (gate_mode == 0) MRS_LAUNCH(0);
        else if (gate_mode == 1) MRS_LAUNCH(1);
        else MRS_LAUNCH(2);
#undef MRS_LAUNCH
        return check_launch("scan_fused_kernel");
    }
    hipLaunchKernelGGL((chunk_state_kernel<T, S4D>), gridA, block, 0, st, h, delta, u, Bm, bc_stride, a_neg,
                       w.h0copy, w.S, w.sumd, Tlen, di, tiles, C, L);
    int rc = check_launch("chunk_state_kernel");
    if (rc) return rc;
#define MRS_LAUNCH(G)                                                                                      \
    hipLaunchKernelGGL((chunk_out_kernel<T, S4D, G>), gridB, block, 0, st, h, y, delta, u, Bm, Cm, bc_stride, \
                       a_neg, D, gate, gate_stride, w.h0copy, w.S, w.sumd, Tlen, di, tiles, C, L)
    if (gate_mode == 0) MRS_LAUNCH(0);
    else if (gate_mode == 1) MRS_LAUNCH(1);
    else MRS_LAUNCH(2);
#undef MRS_LAUNCH
    return check_launch("chunk_out_kernel");
}

template <typename T>
static int launch_split(hipStream_t st, bool s4d, int gate_mode, float *h, void *y, const void *delta,
                        const void *u, const void *Bm, const void *Cm, int64_t bc_stride,
                        const float *a_neg, const float *D, const void *gate, int64_t gate_stride, float *ws, SplitPlan plan,
                        int batch, int Tlen, int di, int one_launch) {
#define MRS_ARGS                                                                                       \
    st, gate_mode, h, (T *)y, (const T *)delta, (const T *)u, (const T *)Bm, (const T *)Cm, bc_stride, \
        a_neg, D, (const T *)gate, gate_stride, ws, plan, batch, Tlen, di, one_launch
    return s4d ? launch_split_s4d<T, true>(MRS_ARGS) : launch_split_s4d<T, false>(MRS_ARGS);
#undef MRS_ARGS
}

static size_t split_workspace_bytes(int batch, int Tlen, int di, int nchunk) {
    return carve_workspace(nullptr, batch, Tlen, di, nchunk).floats * sizeof(float);
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

extern "C" size_t mrs_ssm_scan_flag_bytes(int batch, int d_inner) {
    (void)batch; (void)d_inner;   // one size for every shape
    return kFlagAreaWords * sizeof(unsigned);
}

extern "C" size_t mrs_ssm_scan_workspace_bytes(int batch, int T, int d_inner, int d_state) {
    if (batch < 1 || T < 1 || d_inner < 1 || d_state != 16) return 256;
    const SplitPlan plan = make_split_plan(batch, T, d_inner);
    if (plan.nchunk < 2) return 256;
    const size_t bytes = split_workspace_bytes(batch, T, d_inner, plan.nchunk);
    return (bytes + 255) & ~(size_t)255;
}

// Shared body of the scan entry points: argument checks, route choice, launches.  `fn` names the caller in messages.
static int scan_dispatch(const char *fn, void *stream, int dtype, float *h, void *y, const void *delta, const void *u,
                         const void *B, const void *C, int64_t bc_stride, const float *a_neg, const float *D,
                         const void *gate, int64_t gate_stride, unsigned flags, void *workspace, size_t workspace_bytes,
                         int batch, int T, int d_inner, int d_state, bool own_buffer = false) {
    int rc = scan_check(fn, dtype, h, y, delta, u, B, C, a_neg, D, bc_stride, batch, T, d_inner, d_state);
    if (rc) return rc;
    int gate_mode = 0;
    if ((flags & MRS_GATE_PREACT) && (flags & MRS_GATE_SILU))
        return fail(MRS_E_SHAPE, "%s: MRS_GATE_PREACT and MRS_GATE_SILU are exclusive", fn);
    if (flags & MRS_GATE_PREACT) gate_mode = 1;
    if (flags & MRS_GATE_SILU) gate_mode = 2;
    if (gate_mode && !gate) return fail(MRS_E_NULL, "%s: gate flag set but gate is NULL", fn);
    if (gate_stride == 0) gate_stride = d_inner;
    if (gate_mode && gate_stride < d_inner) return fail(MRS_E_SHAPE, "%s: gate_stride=%lld < d_inner=%d", fn, (long long)gate_stride, d_inner);
    const bool s4d = (flags & MRS_A_S4D_REAL) != 0;
    hipStream_t st = as_stream(stream);
    if ((flags & MRS_FORCE_SEQUENTIAL) && (flags & MRS_FORCE_PARALLEL))
        return fail(MRS_E_SHAPE, "%s: MRS_FORCE_SEQUENTIAL and MRS_FORCE_PARALLEL are exclusive", fn);
    // T-split route: d_state 16, rows of B/C readable as packed dwords, a workspace to put the chunk summaries in.
    const size_t es = (dtype == MRS_F32) ? 4 : 2;
    const bool rows_ok = aligned(B, 4) && aligned(C, 4) && (bc_stride * es) % 4 == 0;
    bool split = d_state == 16 && rows_ok && workspace && !(flags & MRS_FORCE_SEQUENTIAL);
    SplitPlan plan = {1, T};
    if (split) {
        plan = make_split_plan(batch, T, d_inner);
        // Up to 256 steps (where the reference's Auto mode takes its serial kernel, src/config.rs:21-37) the single
        // pass is kept when it fills the machine on its own; with few (batch row, channel tile) pairs the serial walk is
        // one wave per pair and a memory round trip per step (636 us for 256 steps at batch 1, d_inner 2048).
        const int64_t pairs = (int64_t)batch * ((d_inner + kWave - 1) / kWave);
        if (plan.nchunk < 2 || (T <= 256 && pairs >= 1024 && !(flags & MRS_FORCE_PARALLEL))) split = false;
    }
    if ((flags & MRS_FORCE_PARALLEL) && !split && d_state == 16 && T >= 64)
        return fail(MRS_E_WORKSPACE, "%s: MRS_FORCE_PARALLEL needs a workspace and 4-byte aligned B/C rows", fn);
    if (split) {
        const size_t need = split_workspace_bytes(batch, T, d_inner, plan.nchunk);
        if (workspace_bytes < need)
            return fail(MRS_E_WORKSPACE, "%s: workspace %zu bytes < %zu needed", fn, workspace_bytes, need);
        if (!aligned(workspace, 256)) return fail(MRS_E_ALIGN, "%s: workspace must be 256-byte aligned", fn);
        // One launch for both passes where it wins: diagonal-real A (the per-step work of the general form hides the second
        // launch already, and its longer waves wait longer on each other: 141 against 135 us at 8 x 2048 x 1536) and at
        // least 2048 waves (a single 4096-step prompt at d_inner 2048 is 60 us in two launches, 63 in one).
        // MRS_FORCE_PARALLEL takes the one launch at any size, MRS_SCAN_TWO_LAUNCHES (flag or environment) never does.
        // The flag area is cleared by a small kernel first unless it is known to be zero (the caller's word, or the
        // library's own buffer, which starts zeroed and is left zeroed by every launch).
        static const bool env_two = [] { const char *e = getenv("MRS_SCAN_TWO_LAUNCHES"); return e && atoi(e) != 0; }();
        const int64_t waves = (int64_t)batch * ((d_inner + kWave - 1) / kWave) * plan.nchunk;
        const bool wins = (s4d && waves >= 2048) || (flags & MRS_FORCE_PARALLEL);
        int one_launch = (env_two || (flags & MRS_SCAN_TWO_LAUNCHES) || !wins || !flags_fit(batch, d_inner)) ? 0
                         : ((own_buffer || (flags & MRS_SCAN_FLAGS_ZERO)) ? 2 : 1);
        MRS_DISPATCH_DTYPE(dtype, T_, return launch_split<T_>(st, s4d, gate_mode, h, y, delta, u, B, C, bc_stride, a_neg, D, gate, gate_stride,
                                                             (float *)workspace, plan, batch, T, d_inner, one_launch));
    }
    MRS_DISPATCH_DTYPE(dtype, T_, return launch_seq<T_>(st, s4d, gate_mode, h, y, delta, u, B, C, bc_stride, a_neg, D, gate, gate_stride, batch, T, d_inner, d_state));
    return MRS_OK;
}

extern "C" int mrs_ssm_scan_fwd_ex(void *stream, int dtype, float *h, void *y, const void *delta,
                                   const void *u, const void *B, const void *C, int64_t bc_stride,
                                   const float *a_neg, const float *D, const void *gate, int64_t gate_stride,
                                   unsigned flags, void *workspace, size_t workspace_bytes, int batch, int T,
                                   int d_inner, int d_state) {
    return scan_dispatch("mrs_ssm_scan_fwd_ex", stream, dtype, h, y, delta, u, B, C, bc_stride, a_neg, D, gate, gate_stride, flags,
                         workspace, workspace_bytes, batch, T, d_inner, d_state);
}

// ---- the scan without any allocation: chunk summaries in a buffer the library itself holds ---------------------------
// File-scope device array, one copy per GPU the library runs on, held until the process ends.  In host code the name is
// only a handle for hipGetSymbolAddress; kernels and every other use get the per-device address looked up below.
constexpr size_t kStaticScanScratchBytes = MRS_SCAN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScanScratchBytes];

constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each GPU, looked up once with that GPU current
static std::mutex g_scratch_mu;

static int static_scratch_for_current_device(const char *fn, void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(MRS_E_HIP, "%s: hipGetDevice: %s", fn, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(MRS_E_HIP, "%s: device ordinal %d outside 0..%d", fn, dev, kMaxDevices - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(MRS_E_HIP, "%s: hipGetSymbolAddress(scratch) on device %d: %s", fn, dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return MRS_OK;
}

extern "C" int mrs_ssm_scan_fwd_static(void *stream, int dtype, float *h, void *y, const void *delta,
                                       const void *u, const void *B, const void *C, int64_t bc_stride,
                                       const float *a_neg, const float *D, const void *gate, int64_t gate_stride,
                                       unsigned flags, int batch, int T, int d_inner, int d_state) {
    const char *fn = "mrs_ssm_scan_fwd_static";
    // argument checks and the size test come first and touch no GPU: a shape whose chunk summaries do not fit is refused,
    // never shrunk
    int rc = scan_check(fn, dtype, h, y, delta, u, B, C, a_neg, D, bc_stride, batch, T, d_inner, d_state);
    if (rc) return rc;
    const size_t need = mrs_ssm_scan_workspace_bytes(batch, T, d_inner, d_state);
    if (need > kStaticScanScratchBytes)
        return fail(MRS_E_WORKSPACE, "%s: this shape needs %zu bytes of chunk summaries, the built-in buffer holds %zu; use mrs_ssm_scan_fwd_ex with a workspace",
                    fn, need, kStaticScanScratchBytes);
    void *ws = nullptr;
    rc = static_scratch_for_current_device(fn, &ws);
    if (rc) return rc;
    // Every float a wave reads from the buffer is written by another wave of the same call (chunk states, step sums);
    // the flags those waves signal with start at zero (a file-scope device array does) and every launch leaves them zero.
    return scan_dispatch(fn, stream, dtype, h, y, delta, u, B, C, bc_stride, a_neg, D, gate, gate_stride, flags, ws,
                         kStaticScanScratchBytes, batch, T, d_inner, d_state, /*own_buffer=*/true);
}

extern "C" int mrs_ssm_scan_fwd(void *stream, int dtype, float *h, void *y, const void *delta,
                                const void *u, const void *B, const void *C, const float *a_neg,
                                const float *D, int batch, int T, int d_inner, int d_state) {
    return mrs_ssm_scan_fwd_ex(stream, dtype, h, y, delta, u, B, C, d_state, a_neg, D, nullptr, 0,
                               MRS_GATE_NONE, nullptr, 0, batch, T, d_inner, d_state);
}
