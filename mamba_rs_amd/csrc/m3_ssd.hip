// Mamba-3 SISO chunked SSD forward on the matrix cores.
//
// Replaces the reference's six-kernel pipeline m3_preprocess_chunks / m3_dA_cumsum /
// m3_chunk_state_fwd / m3_state_passing_fwd / m3_chunk_scan_fwd /
// m3_writeback_parallel_states (kernels/mamba3_chunked.cu:57-419) with ONE kernel:
// a workgroup owns a (batch row, head) and walks its 64-step chunks in order, so the
// inter-chunk state never leaves registers, K_scaled / qk_dot / dA_cumsum / chunk states
// are never written to memory, and Q, K, x are read once and y written once.
//
// Per chunk (t, s index the 64 steps, n the state, p the head dimension):
//   G^T[s,t] = sum_n K[s,n] Q[t,n]                                   (MFMA, K = n)
//   P[t,s]   = G[t,s] scale[s] exp(dA[t]-dA[s])   (s <  t)
//            = D + gamma[t] G[t,t]                (s == t)  -- the D / qk_dot skip term
//            = 0                                  (s >  t)
//   y[t,p]   = exp(dA[t]) sum_n Q[t,n] S[p,n]  +  sum_s P[t,s] x[s,p]   (MFMA, K = n then K = s)
//   S^T[n,p] = exp(dA_end) S^T[n,p] + sum_t K[t,n] (w[t] x[t,p]),  w[t] = exp(dA_end-dA[t]) scale[t]
// with gamma = dt trap, scale[t] = gamma[t] + dt[t+1](1-trap[t+1]), dA = cumsum(a dt) in the chunk.
//
// When batch*heads alone cannot fill 256 compute units the sequence is also cut into
// super-chunks (a run of consecutive chunks): a state-only pass of the same kernel (no Q, no y)
// leaves each super-chunk's locally accumulated state and total log-decay in a workspace, and the
// full pass then starts every super-chunk from  sum_k exp(sum_{k<m<sc} dA_m) S_k  -- the same
// composition law as between chunks -- so all super-chunks of a (row, head) run concurrently.
//
// Wave w of the workgroup owns the 16 columns p in [16w, 16w+16) of y and of the state.
// Operand layouts are chosen so that no accumulator is ever transposed: G is produced
// transposed (A = K rows, B = Q rows) which leaves P directly in A-operand layout, and the
// state is kept as S^T accumulator tiles, which is B-operand layout for Q S^T.
// v_mfma_f32_16x16x16 (bf16 or f16 inputs, f32 accumulate): lane l holds A[m=l%16][k=4(l/16)..+3],
// B[k=4(l/16)..+3][n=l%16], and C/D[m=4(l/16)+i][n=l%16], i = 0..3.
#include "common.hpp"
#include <stdlib.h>
#include <algorithm>

namespace mrs {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

constexpr int kCS = 64;  // chunk size (the reference's CHUNK_SIZE, src/mamba3_siso/gpu/state.rs:97)
template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    __device__ static __forceinline__ v4f mma(uint2 a, uint2 b, v4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(v4s, a), __builtin_bit_cast(v4s, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint2 pack(float a, float b, float c, float d) {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        b2 lo = {(__bf16)a, (__bf16)b}, hi = {(__bf16)c, (__bf16)d};
        return make_uint2(__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi));
    }
    __device__ static __forceinline__ void unpack(uint2 v, float (&o)[4]) {
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
    }
};
template <> struct Mma<f16_t> {
    __device__ static __forceinline__ v4f mma(uint2 a, uint2 b, v4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(v4h, a), __builtin_bit_cast(v4h, b), c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint2 pack(float a, float b, float c, float d) {
        v4h v = {(_Float16)a, (_Float16)b, (_Float16)c, (_Float16)d};
        return __builtin_bit_cast(uint2, v);
    }
    __device__ static __forceinline__ void unpack(uint2 v, float (&o)[4]) {
        const v4h h = __builtin_bit_cast(v4h, v);
        o[0] = (float)h.x; o[1] = (float)h.y; o[2] = (float)h.z; o[3] = (float)h.w;
    }
};

constexpr int kPad = 8;  // halfword padding of LDS rows: 64-wide rows are 36 dwords, which spreads the 16 rows x 4 dwords that
                         // half a wave reads as operand fragments over all banks (measured: with 40-dword rows half of
                         // the LDS cycles of the pass were bank conflicts; an XOR swizzle of unpadded rows gave the same
                         // conflict count as this padding and cost address arithmetic)

template <int HD, int DS> struct alignas(16) SsdSmem {
    alignas(16) uint16_t Qs[kCS][DS + kPad];       // Q rows
    alignas(16) uint16_t Ks[kCS][DS + kPad];       // K rows
    alignas(16) uint16_t Xs[kCS][HD + kPad];       // x rows of this head
    alignas(16) float sc[5][kCS];                  // dA, scale, gamma, exp(dA), w
    float dAend;                                   // the chunk's total log-decay
    alignas(16) uint2 Ps[10][kWave];               // the 10 causal 16x16 tiles of P as A-operand fragments, by lane
    alignas(16) float gb[2][DS];                   // GEN: the head's B and C biases
};

// A 16x16x16 operand fragment whose contraction index runs along the ROWS of a row-major LDS tile (K^T and x as the
// state update and P x need them): ds_read_b64_tr_b16 hands lane (lr, lg) the four values tile[k0 + 4 lg + e][m0 + lr],
// e = 0..3, when the lanes of each 16-lane group point at the 4-row x 16-column block that holds them -- lane lr at
// row lr / 4, columns 4 (lr % 4)...  No transposed copy of the tile is kept.
__device__ __forceinline__ uint2 lds_frag_tr(const uint16_t *tile, int ld, int k0, int m0, int lr, int lg) {
    const uint16_t *p = tile + (k0 + 4 * lg + (lr >> 2)) * ld + m0 + 4 * (lr & 3);
    const v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s __attribute__((address_space(3))) *)p);
    return __builtin_bit_cast(uint2, v);
}

// Super-chunk split of one launch: nsc super-chunks of cps chunks each; the three buffers live in
// the caller's workspace (null when nsc == 1).
struct SsdSplit {
    float *Sloc;    // [batch*nh][nsc-1][HD][DS]  state accumulated inside super-chunk k (k = 0 includes the carried-in state)
    float *dAtot;   // [batch*nh][nsc-1]          sum of a*dt over super-chunk k
    float *Sinit;   // [batch*nh][HD][DS]         the carried-in state, saved before the last super-chunk overwrites ssm
    int nsc, cps;
    // engine-only extra: x rows may sit inside wider rows (read in place from a projection)
    int64_t x_stride;     // elements between consecutive rows of x (d_inner for a dense x)
    // engine-only extra: K and Q formed inside the kernel (GEN), K = rot(angle, bn + b_bias[h]), Q = rot(angle, cn + c_bias[h]);
    // bn / cn: the normalised and weighted B / C rows in the storage type, g_bcs elements apart; angle [batch, T, nh, g_nr];
    // the first g_nr pairs of a row are rotated (g_nr a multiple of 4)
    const void *g_bn, *g_cn;
    const float *g_ang, *g_bb, *g_cb;
    int64_t g_bcs;
    int g_nr;
    int g_groups;         // batch rows x super-chunks of the launch (set per launch)
    int g_head_major;     // dt, trap, a_val are [batch, nh, T] and the angles [batch, nh, T, g_nr]
    // engine-only extra: y leaves multiplied by silu(z), z rows g_zs elements apart in the storage type (GATE)
    const void *g_z;
    int64_t g_zs;
};

// Cross-lane moves on the data-parallel-primitive path of the vector ALU (no LDS round trip, unlike the shuffle
// builtins): an inclusive sum over the 64 lanes -- shifts of 1, 2, 4, 8 inside each row of 16 lanes, then the last lane of rows 0 and 2 added to rows 1 and 3, then lane 31 to the
// upper half.  Lanes without a source add zero.
template <int CTRL, int ROWS> __device__ __forceinline__ float dpp_add(float v) {
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROWS, 0xf, false));
}
__device__ __forceinline__ float wave_inclusive_sum(float v) {
    v = dpp_add<0x111, 0xf>(v);   // row_shr:1
    v = dpp_add<0x112, 0xf>(v);   // row_shr:2
    v = dpp_add<0x114, 0xf>(v);   // row_shr:4
    v = dpp_add<0x118, 0xf>(v);   // row_shr:8
    v = dpp_add<0x142, 0xa>(v);   // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xc>(v);   // row_bcast:31 into rows 2 and 3
    return v;
}

// Buffer resources for the per-chunk traffic of a workgroup: the address of an access is a scalar base, a scalar offset
// that moves with the chunk and a 32-bit lane offset fixed for the whole walk, so the walk costs no vector integer
// work (64-bit multiplies and adds per access otherwise).  A slab (one batch row of a tensor) stays below 2^31 bytes;
// the launcher checks that.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t slab_rsrc(const void *base, int64_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 slab_ld128(__amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff) {
    return __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
__device__ __forceinline__ float slab_ldf(__amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}

template <typename T, int HD, int DS, bool STATE_ONLY, bool GEN, bool GATE = false>
__global__ __launch_bounds__(HD * 4) __attribute__((amdgpu_waves_per_eu(HD == 64 ? 3 : 1))) void m3_ssd_kernel(
    float *__restrict__ ssm, float *__restrict__ kst, float *__restrict__ vst, T *__restrict__ y,
    const T *__restrict__ x, const T *__restrict__ K, const T *__restrict__ Q,
    const float *__restrict__ dt, const float *__restrict__ trap, const float *__restrict__ a_val,
    const float *__restrict__ Dp, SsdSplit sp, int Tlen, int nh, int carry) {
    constexpr int NW = HD / 16, NTHR = NW * 64, KN = DS / 16;
    constexpr int VPR = DS / 8;                    // 16-byte vectors per Q/K row
    constexpr int NVEC = kCS * VPR;                // vectors per tile
    constexpr int NV = (NVEC + NTHR - 1) / NTHR;   // vectors per thread per tile
    __shared__ SsdSmem<HD, DS> sm;

    const int nscg = STATE_ONLY ? sp.nsc - 1 : sp.nsc;   // the state-only pass skips the last super-chunk
    int b, h, sc;
    if constexpr (GEN) {
        // Workgroups go to the 8 L2 domains of the chip round-robin by index.  The heads of one (batch row, super-chunk)
        // read the same B / C rows, and neighbouring heads share the cache lines of the angle rows: all of them take
        // indices of one residue mod 8, so they meet in one L2.  The grid is padded to whole rounds of 8 groups.
        const int slot = blockIdx.x >> 3, g = (slot / nh) * 8 + (blockIdx.x & 7);
        if (g >= sp.g_groups) return;   // padding: the whole workgroup leaves before any barrier
        h = slot % nh; b = g / nscg; sc = g - b * nscg;
    } else {
        const int bhi = blockIdx.x / nscg;
        sc = blockIdx.x - bhi * nscg; b = bhi / nh; h = bhi - b * nh;
    }
    const int tid = threadIdx.x, l = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave index, in a scalar register: what depends on it alone branches without masks
    const int lr = l & 15, lg = l >> 4;            // fragment row/col index and k-group
    const int di = nh * HD;
    const int64_t bh = (int64_t)b * nh + h;
    const float Dh = Dp[h];
    const int nchunks = (Tlen + kCS - 1) / kCS;
    const int c_begin = sc * sp.cps, c_end = min(nchunks, c_begin + sp.cps);
    const int64_t srow = (bh * HD + 16 * w + lr) * DS + 4 * lg;   // this lane's state elements, + 16 jn

    // ---- running state S^T as accumulator tiles: lane holds S[p=16w+lr][n=16jn+4lg+i] ----
    v4f St[KN];
#pragma unroll
    for (int jn = 0; jn < KN; jn++) St[jn] = (v4f){0.f, 0.f, 0.f, 0.f};
    if (sc == 0) {
        if (carry && !STATE_ONLY && sp.nsc > 1) {
#pragma unroll
            for (int jn = 0; jn < KN; jn++) {
                const float4 s = *reinterpret_cast<const float4 *>(sp.Sinit + srow + 16 * jn);
                St[jn] = (v4f){s.x, s.y, s.z, s.w};
            }
        } else if (carry) {
            // S_in = ssm + dt_0 (1 - trap_0) v_in (x) k_in : the beta term of step 0, which belongs to the carried state
            const int64_t t0row = (GEN && sp.g_head_major) ? ((int64_t)b * nh + h) * Tlen : (int64_t)b * Tlen * nh + h;
            const float sgm1 = dt[t0row] * (1.0f - trap[t0row]);
            const float vin = vst[bh * HD + 16 * w + lr];
#pragma unroll
            for (int jn = 0; jn < KN; jn++) {
                const float4 s = *reinterpret_cast<const float4 *>(ssm + srow + 16 * jn);
                const float4 kin = *reinterpret_cast<const float4 *>(kst + bh * DS + 16 * jn + 4 * lg);
                St[jn] = (v4f){fmaf(sgm1 * vin, kin.x, s.x), fmaf(sgm1 * vin, kin.y, s.y), fmaf(sgm1 * vin, kin.z, s.z),
                               fmaf(sgm1 * vin, kin.w, s.w)};
                if (STATE_ONLY)
                    *reinterpret_cast<float4 *>(sp.Sinit + srow + 16 * jn) = make_float4(St[jn][0], St[jn][1], St[jn][2], St[jn][3]);
            }
        }
    }
    float dAsum = 0.0f;

    // ---- global -> register prefetch of one chunk ----
    struct Pre {
        // the Q / K vectors of the thread (GEN: of the rows they are formed from, and the 4 angles of their pairs)
        uint4 rq[NV], rk[NV], rang[GEN ? NV : 1], rx[2], rz[GATE ? 2 : 1];   // rz: the gate rows of the chunk, laid out like x
        float rdt, rtr, ra, rdtn, rtrn;   // wave 0 only.  lane = step: dt, trap, a of the step; dt, trap of the step after the chunk (every lane the same)
    };
    const unsigned es = (unsigned)sizeof(T);
    const int64_t kq_row = (int64_t)nh * DS;   // elements between consecutive steps of Q / K
    const __amdgpu_buffer_rsrc_t qbuf = slab_rsrc(Q + ((int64_t)b * Tlen * nh + h) * DS, ((int64_t)Tlen * kq_row - h * DS) * es);
    const __amdgpu_buffer_rsrc_t kbuf = slab_rsrc(K + ((int64_t)b * Tlen * nh + h) * DS, ((int64_t)Tlen * kq_row - h * DS) * es);
    const __amdgpu_buffer_rsrc_t xbuf =
        slab_rsrc(x + (int64_t)b * Tlen * sp.x_stride + h * HD, ((int64_t)Tlen * sp.x_stride - h * HD) * es);
    // step scalars of this head: a row of nh apart ([batch, T, nh], the reference's layout) or next to each other
    const bool hm = GEN && sp.g_head_major;
    const int sc_step = hm ? 1 : nh;               // floats between consecutive steps
    const int64_t sc_base = hm ? ((int64_t)b * nh + h) * Tlen : (int64_t)b * Tlen * nh + h;
    const int64_t sc_bytes = hm ? (int64_t)Tlen * 4 : ((int64_t)Tlen * nh - h) * 4;
    const __amdgpu_buffer_rsrc_t dtbuf = slab_rsrc(dt + sc_base, sc_bytes);
    const __amdgpu_buffer_rsrc_t trbuf = slab_rsrc(trap + sc_base, sc_bytes);
    const __amdgpu_buffer_rsrc_t abuf = slab_rsrc(a_val + sc_base, sc_bytes);
    const __amdgpu_buffer_rsrc_t ybuf = slab_rsrc(y + (int64_t)b * Tlen * di + h * HD, ((int64_t)Tlen * di - h * HD) * es);
    unsigned kq_voff[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int vi = tid + v * NTHR, row = vi / VPR, col = (vi % VPR) * 8;
        kq_voff[v] = vi < NVEC ? (unsigned)(row * (int)kq_row + col) * es : 0u;   // lanes past the tile read a valid element and drop it
    }
    // GEN: the same (row, 8 columns) items read bn / cn (f32) and the 4 angles of their pairs instead of K / Q
    const int g_col = (tid % VPR) * 8;             // the thread's columns, the same for each of its vectors
    const bool g_rot = g_col < 2 * sp.g_nr;        // its pairs are rotated (all four or none: g_nr is a multiple of 4)
    const __amdgpu_buffer_rsrc_t bnbuf = slab_rsrc(GEN ? (const T *)sp.g_bn + (int64_t)b * Tlen * sp.g_bcs : nullptr, GEN ? (int64_t)Tlen * sp.g_bcs * es : 0);
    const __amdgpu_buffer_rsrc_t cnbuf = slab_rsrc(GEN ? (const T *)sp.g_cn + (int64_t)b * Tlen * sp.g_bcs : nullptr, GEN ? (int64_t)Tlen * sp.g_bcs * es : 0);
    const int ang_step = hm ? sp.g_nr : nh * sp.g_nr;   // floats between the angle rows of consecutive steps
    const __amdgpu_buffer_rsrc_t angbuf =
        slab_rsrc(GEN ? sp.g_ang + (hm ? ((int64_t)b * nh + h) * Tlen : (int64_t)b * Tlen * nh + h) * sp.g_nr : nullptr,
                  GEN ? (hm ? (int64_t)Tlen : (int64_t)Tlen * nh - h) * sp.g_nr * 4 : 0);
    unsigned bc_voff[NV], ang_voff[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int vi = tid + v * NTHR, row = vi / VPR;
        bc_voff[v] = GEN && vi < NVEC ? (unsigned)(row * (int)sp.g_bcs + g_col) * es : 0u;
        ang_voff[v] = GEN && vi < NVEC && g_rot ? (unsigned)(row * ang_step + g_col / 2) * 4u : 0u;
    }
    if (GEN) {   // visible to every wave after the barrier at the top of the first chunk
        for (int n = tid; n < DS; n += NTHR) { sm.gb[0][n] = sp.g_bb[h * DS + n]; sm.gb[1][n] = sp.g_cb[h * DS + n]; }
    }
    // the x tile (64 steps x HD) is fetched like the Q / K tiles, whole rows by neighbouring lanes: HD / 8 vectors a row,
    // two vectors a thread for any HD (a lane fetching its own step's row piece touched 64 cache lines per instruction)
    constexpr int VPRX = HD / 8;
    unsigned x_voff[2];
    int x_row[2], x_col[2];
#pragma unroll
    for (int v = 0; v < 2; v++) {
        const int vi = tid + v * NTHR;
        x_row[v] = vi / VPRX; x_col[v] = (vi % VPRX) * 8;
        x_voff[v] = (unsigned)(x_row[v] * (int)sp.x_stride + x_col[v]) * es;
    }
    const unsigned sc_voff = (unsigned)l * (unsigned)sc_step * 4u;
    const __amdgpu_buffer_rsrc_t zbuf = slab_rsrc(GATE ? (const T *)sp.g_z + (int64_t)b * Tlen * sp.g_zs + h * HD : nullptr,
                                                  GATE ? ((int64_t)Tlen * sp.g_zs - h * HD) * es : 0);
    unsigned z_voff[2];
#pragma unroll
    for (int v = 0; v < 2; v++) z_voff[v] = GATE ? (unsigned)(x_row[v] * (int)sp.g_zs + x_col[v]) * es : 0u;
    unsigned y_voff[2];   // the y tile leaves like the x tile comes in: whole rows by neighbouring lanes, 16 bytes a lane
#pragma unroll
    for (int v = 0; v < 2; v++) y_voff[v] = (unsigned)(x_row[v] * di + x_col[v]) * es;
    // Accesses past the end of the batch row (the tail of a last, partial chunk) fall outside the resources: loads give
    // zero and stores are dropped by the bounds check, which covers the vector offset -- so the chunk's offset goes there.
    auto prefetch = [&](Pre &r, int c) {
        const int t0 = c * kCS;
        const unsigned kq_c = (unsigned)t0 * (unsigned)kq_row * es, x_c = (unsigned)t0 * (unsigned)sp.x_stride * es, sc_c = (unsigned)t0 * (unsigned)sc_step * 4u;
        // The step scalars go first: loads return in order, and the compiler moves the first uses of these small values
        // ahead of the next request, so whoever waits for them must not wait for the tiles requested after them as well.
        // Wave 0 alone fetches them: a step's scalars of one head are 4 bytes in a row of nh, so each of these loads
        // touches as many cache lines as it has lanes -- with every wave fetching all five arrays the scalars were most of
        // the workgroup's memory requests (measured with the loads taken out: state-only pass 39 -> 25 us, full pass
        // 70 -> 59 us on the route that forms K and Q).  The step after the chunk is one address for all lanes.
        if (w == 0) {
            r.rdt = slab_ldf(dtbuf, sc_voff + sc_c, 0);
            r.rtr = slab_ldf(trbuf, sc_voff + sc_c, 0);
            r.ra = slab_ldf(abuf, sc_voff + sc_c, 0);
            r.rdtn = slab_ldf(dtbuf, sc_c + (unsigned)(kCS * sc_step) * 4u, 0);   // zero past the row
            r.rtrn = slab_ldf(trbuf, sc_c + (unsigned)(kCS * sc_step) * 4u, 0);
        }
        if constexpr (GEN) {
            const unsigned bc_c = (unsigned)t0 * (unsigned)sp.g_bcs * es, ang_c = (unsigned)t0 * (unsigned)ang_step * 4u;
#pragma unroll
            for (int v = 0; v < NV; v++) {
                if (!STATE_ONLY) r.rq[v] = slab_ld128(cnbuf, bc_voff[v] + bc_c, 0);
                r.rk[v] = slab_ld128(bnbuf, bc_voff[v] + bc_c, 0);
                r.rang[v] = slab_ld128(angbuf, ang_voff[v] + ang_c, 0);   // lanes without rotated pairs: some angle, not used
            }
        } else {
#pragma unroll
            for (int v = 0; v < NV; v++) {
                if (!STATE_ONLY) r.rq[v] = slab_ld128(qbuf, kq_voff[v] + kq_c, 0);
                r.rk[v] = slab_ld128(kbuf, kq_voff[v] + kq_c, 0);
            }
        }
        r.rx[0] = slab_ld128(xbuf, x_voff[0] + x_c, 0);
        r.rx[1] = slab_ld128(xbuf, x_voff[1] + x_c, 0);
        if constexpr (GATE) {
            const unsigned z_c = (unsigned)t0 * (unsigned)sp.g_zs * es;
            r.rz[0] = slab_ld128(zbuf, z_voff[0] + z_c, 0);
            r.rz[1] = slab_ld128(zbuf, z_voff[1] + z_c, 0);
        }
    };

    // One chunk from the registers of `r`; once they are in LDS the chunk c_next is requested into them.
    auto chunk = [&](Pre &r, int c, int c_next) {
        const int t0 = c * kCS;
        // Issue priority falls with progress (after 1/2, 3/4, 7/8 of the walk): the arbiter of a SIMD serves its oldest wave
        // first, so the workgroups sharing a compute unit would otherwise finish one after the other and the last one run
        // alone; with the one that is behind served first they finish together.
        {
            const int done = c - c_begin, total = c_end - c_begin;
            if (done * 8 >= total * 7) __builtin_amdgcn_s_setprio(0);
            else if (done * 4 >= total * 3) __builtin_amdgcn_s_setprio(1);
            else if (done * 2 >= total) __builtin_amdgcn_s_setprio(2);
            else __builtin_amdgcn_s_setprio(3);
        }
        lds_barrier();  // every wave is done reading the previous chunk's tiles (LDS only: y stores and the prefetch stay in flight)
        // ---- registers -> LDS ----
#pragma unroll
        for (int v = 0; v < NV; v++) {
            const int vi = tid + v * NTHR, row = vi / VPR, col = (vi % VPR) * 8;
            if (vi >= NVEC) continue;
            if constexpr (GEN) {
                // K = rot(bn + b_bias), Q = rot(cn + c_bias): pairs (2j, 2j+1), j < g_nr, turned by the step's angle
                // (hardware sine / cosine: angles lie in [0, 2 pi), the results are stored in 16 bits); lanes whose
                // pairs are not rotated turn by zero
                const float4 an = __builtin_bit_cast(float4, r.rang[v]);
                const float ang[4] = {g_rot ? an.x : 0.f, g_rot ? an.y : 0.f, g_rot ? an.z : 0.f, g_rot ? an.w : 0.f};
                float sn[4], cs[4];
#pragma unroll
                for (int pr = 0; pr < 4; pr++) { sn[pr] = __sinf(ang[pr]); cs[pr] = __cosf(ang[pr]); }
                auto form = [&](const uint4 &raw, const float *bias) {
                    const float4 b0 = *reinterpret_cast<const float4 *>(bias + col), b1 = *reinterpret_cast<const float4 *>(bias + col + 4);
                    float v0[4], v1[4];
                    Mma<T>::unpack(make_uint2(raw.x, raw.y), v0);
                    Mma<T>::unpack(make_uint2(raw.z, raw.w), v1);
                    const float k[8] = {v0[0] + b0.x, v0[1] + b0.y, v0[2] + b0.z, v0[3] + b0.w, v1[0] + b1.x, v1[1] + b1.y, v1[2] + b1.z, v1[3] + b1.w};
                    float o[8];
#pragma unroll
                    for (int pr = 0; pr < 4; pr++) {
                        o[2 * pr] = cs[pr] * k[2 * pr] - sn[pr] * k[2 * pr + 1];
                        o[2 * pr + 1] = sn[pr] * k[2 * pr] + cs[pr] * k[2 * pr + 1];
                    }
                    const uint2 p0 = Mma<T>::pack(o[0], o[1], o[2], o[3]), p1 = Mma<T>::pack(o[4], o[5], o[6], o[7]);
                    return make_uint4(p0.x, p0.y, p1.x, p1.y);
                };
                if (!STATE_ONLY) *reinterpret_cast<uint4 *>(&sm.Qs[row][col]) = form(r.rq[v], sm.gb[1]);
                *reinterpret_cast<uint4 *>(&sm.Ks[row][col]) = form(r.rk[v], sm.gb[0]);
            } else {
                if (!STATE_ONLY) *reinterpret_cast<uint4 *>(&sm.Qs[row][col]) = r.rq[v];
                *reinterpret_cast<uint4 *>(&sm.Ks[row][col]) = r.rk[v];
            }
        }
        *reinterpret_cast<uint4 *>(&sm.Xs[x_row[0]][x_col[0]]) = r.rx[0];
        *reinterpret_cast<uint4 *>(&sm.Xs[x_row[1]][x_col[1]]) = r.rx[1];
        uint4 zc[GATE ? 2 : 1];   // this chunk's gate rows: the registers of `r` take the next chunk's below
        if constexpr (GATE) { zc[0] = r.rz[0]; zc[1] = r.rz[1]; }
        // ---- per-step scalars, lane = step (wave 0) ----
        if (w == 0) {
            // dt, trap of the step after this one: the next lane's, and for the last lane the step after the chunk
            float dtn = __shfl_down(r.rdt, 1), trn = __shfl_down(r.rtr, 1);
            if (l == kCS - 1) { dtn = r.rdtn; trn = r.rtrn; }
            if (t0 + l + 1 >= Tlen) { dtn = 0.f; trn = 1.f; }       // no step after the last one
            const float gam = r.rdt * r.rtr;
            const float scl = fmaf(dtn, 1.0f - trn, gam);
            const float dA = wave_inclusive_sum(r.ra * r.rdt);   // cumulative log-decay over the 64 steps
            const float tot = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, dA), 63));
            sm.sc[0][l] = dA;
            sm.sc[1][l] = scl;
            sm.sc[2][l] = gam;
            sm.sc[3][l] = fast_exp2(dA * kLog2e);
            sm.sc[4][l] = fast_exp2((tot - dA) * kLog2e) * scl;
            if (l == 0) sm.dAend = tot;
        }
        lds_barrier();  // tiles and scalars visible to every wave
        const float dAend = sm.dAend;
        if (c_next < c_end) prefetch(r, c_next);
        dAsum += dAend;

        // ---- x fragments: lane holds x[t=16kt+4lg+i][p=16w+lr]; also scaled by w[t] for the state update ----
        uint2 xf[4], xwf[4];
#pragma unroll
        for (int kt = 0; kt < 4; kt++) {
            xf[kt] = lds_frag_tr(&sm.Xs[0][0], HD + kPad, 16 * kt, 16 * w, lr, lg);
            const float4 wv = *reinterpret_cast<const float4 *>(&sm.sc[4][16 * kt + 4 * lg]);
            float xv[4];
            Mma<T>::unpack(xf[kt], xv);
            xwf[kt] = Mma<T>::pack(xv[0] * wv.x, xv[1] * wv.y, xv[2] * wv.z, xv[3] * wv.w);
        }
        // ---- entering state as B-operand fragments (16-bit) ----
        uint2 Sf[KN];
#pragma unroll
        for (int jn = 0; jn < KN; jn++) Sf[jn] = Mma<T>::pack(St[jn][0], St[jn][1], St[jn][2], St[jn][3]);

        if (!STATE_ONLY) {
            // ---- P tiles: P does not depend on p, so the waves split the 10 causal tiles and share them through LDS ----
#pragma unroll
            for (int it = 0; it < 4; it++) {
#pragma unroll
                for (int js = 0; js <= it; js++) {
                    const int tix = it * (it + 1) / 2 + js;
                    if ((tix % NW) != w) continue;
                    // G^T tile: rows s = 16js+4lg+i, cols t = 16it+lr
                    v4f g = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kk = 0; kk < KN; kk++) {
                        const uint2 kf = *reinterpret_cast<const uint2 *>(&sm.Ks[16 * js + lr][16 * kk + 4 * lg]);
                        const uint2 qf = *reinterpret_cast<const uint2 *>(&sm.Qs[16 * it + lr][16 * kk + 4 * lg]);
                        g = Mma<T>::mma(kf, qf, g);
                    }
                    const float dAt = sm.sc[0][16 * it + lr];
                    const float4 dAs = *reinterpret_cast<const float4 *>(&sm.sc[0][16 * js + 4 * lg]);
                    const float4 scs = *reinterpret_cast<const float4 *>(&sm.sc[1][16 * js + 4 * lg]);
                    const float das[4] = {dAs.x, dAs.y, dAs.z, dAs.w}, sc4[4] = {scs.x, scs.y, scs.z, scs.w};
                    const float gam_t = (js == it) ? sm.sc[2][16 * it + lr] : 0.f;
                    float pv[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float dec = fast_exp2((dAt - das[i]) * kLog2e);   // above the diagonal: dropped below, whatever it is
                        pv[i] = g[i] * sc4[i] * dec;
                        if (js == it) {  // diagonal tile: strict causality, skip term on the diagonal (selects, no branches)
                            const int s = 4 * lg + i;
                            const float dg = fmaf(gam_t, g[i], Dh);
                            pv[i] = s > lr ? 0.f : (s == lr ? dg : pv[i]);
                        }
                    }
                    sm.Ps[tix][l] = Mma<T>::pack(pv[0], pv[1], pv[2], pv[3]);  // A operand: P[t=lr][s=4lg+i]
                }
            }
        }
        // ---- state update: S^T[n,p] = exp(dA_end) S^T + K^T (w x) ----
        const float decay = fast_exp2(dAend * kLog2e);
#pragma unroll
        for (int jn = 0; jn < KN; jn++) {
            v4f s = St[jn] * decay;
#pragma unroll
            for (int kt = 0; kt < 4; kt++) {
                const uint2 ktf = lds_frag_tr(&sm.Ks[0][0], DS + kPad, 16 * kt, 16 * jn, lr, lg);   // K^T[n = 16 jn + lr][t = 16 kt + 4 lg + e]
                s = Mma<T>::mma(ktf, xwf[kt], s);
            }
            St[jn] = s;
        }
        if (!STATE_ONLY) {
            lds_barrier();  // P tiles visible; the next chunk's prefetch, issued above, keeps running under the products below
#pragma unroll
            for (int it = 0; it < 4; it++) {
                // y_off = exp(dA[t]) * Q S_in^T     (acc rows t = 16it+4lg+i, cols p = 16w+lr)
                v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < KN; kk++) {
                    const uint2 qf = *reinterpret_cast<const uint2 *>(&sm.Qs[16 * it + lr][16 * kk + 4 * lg]);
                    acc = Mma<T>::mma(qf, Sf[kk], acc);
                }
                {
                    const float4 e = *reinterpret_cast<const float4 *>(&sm.sc[3][16 * it + 4 * lg]);
                    acc[0] *= e.x; acc[1] *= e.y; acc[2] *= e.z; acc[3] *= e.w;
                }
#pragma unroll
                for (int js = 0; js <= it; js++) acc = Mma<T>::mma(sm.Ps[it * (it + 1) / 2 + js][l], xf[js], acc);
                // y rows t = 16it+4lg+i, column p = 16w+lr into the tile that held x (its fragments are in registers since
                // the second barrier): a lane's four values are 2 bytes each in four different rows, and stored to memory
                // like that they were 32-byte pieces, sixteen instructions a wave
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const T yv = (T)acc[i];
                    sm.Xs[16 * it + 4 * lg + i][16 * w + lr] = __builtin_bit_cast(uint16_t, yv);
                }
            }
            lds_barrier();  // the y tile is complete
#pragma unroll
            for (int v = 0; v < 2; v++) {   // rows past the sequence are dropped by the bounds check
                uint4 yv = *reinterpret_cast<const uint4 *>(&sm.Xs[x_row[v]][x_col[v]]);
                if constexpr (GATE) {   // y * silu(z), rounded like the separate gate pass rounds it (y to the storage type first)
                    float yf[8], zf[8];
                    Mma<T>::unpack(make_uint2(yv.x, yv.y), *reinterpret_cast<float(*)[4]>(yf));
                    Mma<T>::unpack(make_uint2(yv.z, yv.w), *reinterpret_cast<float(*)[4]>(yf + 4));
                    Mma<T>::unpack(make_uint2(zc[v].x, zc[v].y), *reinterpret_cast<float(*)[4]>(zf));
                    Mma<T>::unpack(make_uint2(zc[v].z, zc[v].w), *reinterpret_cast<float(*)[4]>(zf + 4));
#pragma unroll
                    for (int e = 0; e < 8; e++) yf[e] *= silu(zf[e]);
                    const uint2 lo = Mma<T>::pack(yf[0], yf[1], yf[2], yf[3]), hi = Mma<T>::pack(yf[4], yf[5], yf[6], yf[7]);
                    yv = make_uint4(lo.x, lo.y, hi.x, hi.y);
                }
                typedef unsigned v4u __attribute__((ext_vector_type(4)));
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, yv), ybuf, y_voff[v] + (unsigned)t0 * (unsigned)di * es, 0, 0);
            }
        }
    };
    // Entering state of super-chunk sc from the local states of the earlier ones (the state-only pass accumulates every
    // later super-chunk from zero):  sum_k exp(sum_{k<m<sc} dA_m) S_k.  The super-chunk's first chunk is requested before
    // this, the local states are fetched four at a time and the decays come from one lane-parallel suffix sum; one state
    // per memory round trip, each behind a dependent scalar load, kept the last super-chunk's workgroup in its prologue
    // for 22 thousand cycles of a walk of 100 thousand.
    auto fold_entering_state = [&]() {
        const int64_t slot0 = bh * (sp.nsc - 1);
        const float mine = l < sc ? sp.dAtot[slot0 + l] : 0.0f;               // nsc <= 32: a wave holds them all
        const float upto = wave_inclusive_sum(mine);
        const float total = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, upto), 63));
        const float dec_l = fast_exp2((total - upto) * kLog2e);               // lane k: exp(sum_{k<m<sc} dA_m)
        constexpr int kFB = 4;
        for (int k0 = sc - 1; k0 >= 0; k0 -= kFB) {
            float4 sv[kFB][KN];
#pragma unroll
            for (int i = 0; i < kFB; i++) {
                const int k = max(k0 - i, 0);                                  // past the front: state 0 again, fetched and not used
                const float *src = sp.Sloc + (slot0 + k) * (HD * DS) + (16 * w + lr) * DS + 4 * lg;
#pragma unroll
                for (int jn = 0; jn < KN; jn++) sv[i][jn] = *reinterpret_cast<const float4 *>(src + 16 * jn);
            }
#pragma unroll
            for (int i = 0; i < kFB; i++) {
                if (k0 - i < 0) continue;                                      // uniform over the workgroup
                const float dec = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, dec_l), k0 - i));
#pragma unroll
                for (int jn = 0; jn < KN; jn++)
                    St[jn] = (v4f){fmaf(dec, sv[i][jn].x, St[jn][0]), fmaf(dec, sv[i][jn].y, St[jn][1]), fmaf(dec, sv[i][jn].z, St[jn][2]),
                                   fmaf(dec, sv[i][jn].w, St[jn][3])};
            }
        }
    };
    if (STATE_ONLY) {
        // The state-only pass does little arithmetic per chunk, so its walk is as long as a memory round trip per chunk
        // allows: two chunks are kept in flight (registers are not scarce here).  The full pass does not have the registers
        // for that: with a second set it spills at the 168 registers that three waves per SIMD allow (measured: 55 -> 93 us).
        Pre ra_, rb_;
        prefetch(ra_, c_begin);
        if (c_begin + 1 < c_end) prefetch(rb_, c_begin + 1);
        for (int c = c_begin; c < c_end; c += 2) {
            chunk(ra_, c, c + 2);
            if (c + 1 < c_end) chunk(rb_, c + 1, c + 3);
        }
    } else {
        Pre r_;
        prefetch(r_, c_begin);
        if (sc > 0) fold_entering_state();
        for (int c = c_begin; c < c_end; c++) chunk(r_, c, c + 1);
    }
    if (STATE_ONLY) {
        const int64_t slot = bh * (sp.nsc - 1) + sc;
        float *dst = sp.Sloc + slot * (HD * DS) + (16 * w + lr) * DS + 4 * lg;
#pragma unroll
        for (int jn = 0; jn < KN; jn++)
            *reinterpret_cast<float4 *>(dst + 16 * jn) = make_float4(St[jn][0], St[jn][1], St[jn][2], St[jn][3]);
        if (tid == 0) sp.dAtot[slot] = dAsum;
        return;
    }
    if (sc != sp.nsc - 1) return;
    // ---- write back: ssm <- S, k_state <- K[T-1], v_state <- x[T-1] ----
#pragma unroll
    for (int jn = 0; jn < KN; jn++)
        *reinterpret_cast<float4 *>(ssm + srow + 16 * jn) = make_float4(St[jn][0], St[jn][1], St[jn][2], St[jn][3]);
    const int64_t last = (int64_t)b * Tlen + (Tlen - 1);
    if constexpr (GEN) {   // K of the last step, as the tiles above form it (rounded to the storage type like a K read from memory)
        for (int n = tid; n < DS; n += NTHR) {
            const int j = n >> 1;
            const T *bnl = (const T *)sp.g_bn + last * sp.g_bcs;
            const float k0 = Store<T>::ld(bnl + 2 * j) + sp.g_bb[h * DS + 2 * j], k1 = Store<T>::ld(bnl + 2 * j + 1) + sp.g_bb[h * DS + 2 * j + 1];
            const float a = j < sp.g_nr ? sp.g_ang[(hm ? ((int64_t)b * nh + h) * Tlen + (Tlen - 1) : last * nh + h) * sp.g_nr + j] : 0.f;
            const float sn = __sinf(a), cs = __cosf(a);
            const T kv = (T)((n & 1) ? sn * k0 + cs * k1 : cs * k0 - sn * k1);
            kst[bh * DS + n] = (float)kv;
        }
    } else {
        for (int n = tid; n < DS; n += NTHR) kst[bh * DS + n] = Store<T>::ld(K + (last * nh + h) * DS + n);
    }
    for (int p = tid; p < HD; p += NTHR) vst[bh * HD + p] = Store<T>::ld(x + last * sp.x_stride + h * HD + p);
}

__global__ void m3_abg_kernel(float *__restrict__ alpha, float *__restrict__ beta, float *__restrict__ gamma,
                              const float *__restrict__ dt, const float *__restrict__ a_val,
                              const float *__restrict__ trap, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float d = dt[i], t = trap[i];
    const float al = fast_exp2(a_val[i] * d * kLog2e);
    alpha[i] = al;
    beta[i] = al * d * (1.0f - t);
    gamma[i] = t * d;
}

__global__ void zero_kernel(float *__restrict__ p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

// Super-chunk plan: enough workgroups to cover the chip about three times over (three workgroups of
// this kernel fit a compute unit), at least two chunks per super-chunk, at most 32 super-chunks.
static void ssd_plan(int batch, int Tlen, int nh, int &nsc, int &cps) {
    const int nchunks = (Tlen + kCS - 1) / kCS;
    int target = 768;
    if (const char *e = getenv("MRS_SSD_TARGET_WGS")) { const int v = atoi(e); if (v > 0) target = v; }
    int64_t want = target / ((int64_t)batch * nh);
    if (want > 32) want = 32;
    if (want > nchunks / 2) want = nchunks / 2;
    if (want <= 1) { nsc = 1; cps = nchunks; return; }
    cps = (nchunks + (int)want - 1) / (int)want;
    nsc = (nchunks + cps - 1) / cps;
}

static size_t ssd_split_bytes(int batch, int nh, int hd, int ds, int nsc, size_t *o_dA, size_t *o_init) {
    if (nsc <= 1) { if (o_dA) *o_dA = 0; if (o_init) *o_init = 0; return 0; }
    const size_t bh = (size_t)batch * nh;
    const size_t sloc = (bh * (nsc - 1) * hd * ds * sizeof(float) + 255) & ~(size_t)255;
    const size_t dat = (bh * (nsc - 1) * sizeof(float) + 255) & ~(size_t)255;
    const size_t sin = (bh * hd * ds * sizeof(float) + 255) & ~(size_t)255;
    if (o_dA) *o_dA = sloc;
    if (o_init) *o_init = sloc + dat;
    return sloc + dat + sin;
}

template <typename T, int HD, int DS>
static void launch_ssd_shape(hipStream_t st, float *ssm, float *kst, float *vst, void *y, const void *x,
                             const void *K, const void *Q, const float *dt, const float *trap,
                             const float *a_val, const float *D, SsdSplit sp, int batch, int Tlen, int nh, int carry) {
    if constexpr (HD == 64 && DS == 64) {   // the one shape the in-kernel K / Q route is built for
        if (sp.g_bn) {
            auto padded = [&](int groups) { return dim3((unsigned)((groups + 7) / 8 * 8 * nh)); };
            if (sp.nsc > 1) {
                sp.g_groups = batch * (sp.nsc - 1);
                hipLaunchKernelGGL((m3_ssd_kernel<T, HD, DS, true, true>), padded(sp.g_groups), dim3(HD * 4), 0, st,
                                   ssm, kst, vst, (T *)y, (const T *)x, (const T *)K, (const T *)Q, dt, trap, a_val, D, sp, Tlen, nh, carry);
            }
            sp.g_groups = batch * sp.nsc;
            if (sp.g_z)
                hipLaunchKernelGGL((m3_ssd_kernel<T, HD, DS, false, true, true>), padded(sp.g_groups), dim3(HD * 4), 0, st, ssm, kst, vst,
                                   (T *)y, (const T *)x, (const T *)K, (const T *)Q, dt, trap, a_val, D, sp, Tlen, nh, carry);
            else
                hipLaunchKernelGGL((m3_ssd_kernel<T, HD, DS, false, true>), padded(sp.g_groups), dim3(HD * 4), 0, st, ssm, kst, vst,
                                   (T *)y, (const T *)x, (const T *)K, (const T *)Q, dt, trap, a_val, D, sp, Tlen, nh, carry);
            return;
        }
    }
    if (sp.nsc > 1)
        hipLaunchKernelGGL((m3_ssd_kernel<T, HD, DS, true, false>), dim3((unsigned)(batch * nh * (sp.nsc - 1))), dim3(HD * 4), 0, st,
                           ssm, kst, vst, (T *)y, (const T *)x, (const T *)K, (const T *)Q, dt, trap, a_val, D, sp, Tlen, nh, carry);
    hipLaunchKernelGGL((m3_ssd_kernel<T, HD, DS, false, false>), dim3((unsigned)(batch * nh * sp.nsc)), dim3(HD * 4), 0, st, ssm, kst, vst,
                       (T *)y, (const T *)x, (const T *)K, (const T *)Q, dt, trap, a_val, D, sp, Tlen, nh, carry);
}

template <typename T>
static int launch_ssd(hipStream_t st, float *ssm, float *kst, float *vst, void *y, const void *x, const void *K,
                      const void *Q, const float *dt, const float *trap, const float *a_val, const float *D,
                      SsdSplit sp, int batch, int Tlen, int nh, int hd, int ds, int carry) {
#define MRS_SHAPE(H, S)                                                                                      \
    if (hd == H && ds == S) {                                                                                \
        launch_ssd_shape<T, H, S>(st, ssm, kst, vst, y, x, K, Q, dt, trap, a_val, D, sp, batch, Tlen, nh, carry); \
        return check_launch("m3_ssd_kernel");                                                                \
    }
    MRS_SHAPE(64, 64) MRS_SHAPE(64, 32) MRS_SHAPE(64, 16)
    MRS_SHAPE(32, 64) MRS_SHAPE(32, 32) MRS_SHAPE(32, 16)
    MRS_SHAPE(16, 64) MRS_SHAPE(16, 32) MRS_SHAPE(16, 16)
#undef MRS_SHAPE
    return fail(MRS_E_SHAPE, "mrs_m3_ssd_fwd: headdim=%d d_state=%d not in {16,32,64}x{16,32,64}", hd, ds);
}

}  // namespace mrs

using namespace mrs;

extern "C" int mrs_m3_compute_abg(void *stream, float *alpha, float *beta, float *gamma, const float *dt,
                                  const float *a_val, const float *trap, int64_t n) {
    if (!alpha || !beta || !gamma || !dt || !a_val || !trap) return fail(MRS_E_NULL, "mrs_m3_compute_abg: null pointer");
    if (n < 1 || n > 0x7fffffffLL * 256) return fail(MRS_E_SHAPE, "mrs_m3_compute_abg: n=%lld", (long long)n);
    hipLaunchKernelGGL(m3_abg_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), alpha, beta, gamma,
                       dt, a_val, trap, n);
    return check_launch("m3_abg_kernel");
}

extern "C" size_t mrs_m3_ssd_workspace_bytes(int batch, int T, int nheads, int headdim, int d_state, int chunk_size) {
    (void)chunk_size;
    if (batch < 1 || T < 1 || nheads < 1 || headdim < 1 || d_state < 1) return 256;
    // the larger of: alpha, beta, gamma for the f32-storage route (sequential kernel); the
    // super-chunk states of the 16-bit route
    const size_t n = (size_t)batch * T * nheads;
    const size_t f32_route = ((3 * n * sizeof(float)) + 255) & ~(size_t)255;
    int nsc, cps;
    ssd_plan(batch, T, nheads, nsc, cps);
    const size_t split = ssd_split_bytes(batch, nheads, headdim, d_state, nsc, nullptr, nullptr);
    return f32_route > split ? f32_route : split;
}

extern "C" int mrs_m3_ssd_fwd(void *stream, int dtype, float *ssm_state, float *k_state, float *v_state, void *y,
                              const void *x, const void *K, const void *Q, const float *dt, const float *trap,
                              const float *a_val, const float *D, void *workspace, size_t workspace_bytes,
                              unsigned flags, int batch, int T, int nheads, int headdim, int d_state,
                              int chunk_size) {
    return mrs::m3_ssd_fwd_ex(stream, dtype, ssm_state, k_state, v_state, y, x, 0, K, Q, dt, trap, a_val, D, workspace,
                              workspace_bytes, flags, batch, T, nheads, headdim, d_state, chunk_size, nullptr);
}

// x_stride = 0 means dense rows (d_inner); a wider stride needs 16-bit storage (the f32 route runs the recurrence kernel).
int mrs::m3_ssd_fwd_ex(void *stream, int dtype, float *ssm_state, float *k_state, float *v_state, void *y, const void *x,
                       int64_t x_stride, const void *K, const void *Q, const float *dt,
                       const float *trap, const float *a_val, const float *D, void *workspace, size_t workspace_bytes,
                       unsigned flags, int batch, int T, int nheads, int headdim, int d_state, int chunk_size, const SsdGenArgs *gen) {
    const char *fn = "mrs_m3_ssd_fwd";
    if (gen) {   // K and Q formed inside the kernel: K and Q themselves are not read
        if (dtype == MRS_F32 || headdim != 64 || d_state != 64 || gen->n_rope % 4 != 0 || 2 * gen->n_rope > d_state || gen->bc_stride % 8 != 0 ||
            !gen->bn || !gen->cn || !gen->angle || !gen->b_bias || !gen->c_bias || !aligned(gen->bn, 16) || !aligned(gen->cn, 16) || !aligned(gen->angle, 16) ||
            (gen->gate && (!aligned(gen->gate, 16) || gen->gate_stride % 8 != 0 || (int64_t)T * gen->gate_stride * 2 >= 0x7fffffffLL)))
            return fail(MRS_E_SHAPE, "%s: in-kernel K / Q needs 16-bit storage, headdim = d_state = 64, rope pairs in fours, aligned rows", fn);
        if ((int64_t)T * std::max<int64_t>(gen->bc_stride, (int64_t)nheads * gen->n_rope) * 4 >= 0x7fffffffLL)
            return fail(MRS_E_SHAPE, "%s: one batch row of the B / C rows or the angles exceeds 2^31 bytes", fn);
        K = Q = x;   // placeholders for the checks below
    }
    const int64_t di_ = (int64_t)nheads * headdim;
    if (x_stride == 0) x_stride = di_;
    if (x_stride < di_) return fail(MRS_E_SHAPE, "%s: row stride below d_inner", fn);
    if (dtype == MRS_F32 && x_stride != di_) return fail(MRS_E_SHAPE, "%s: strided x needs 16-bit storage", fn);
    if (x_stride % 8 != 0) return fail(MRS_E_ALIGN, "%s: x row stride must be a multiple of 8 elements", fn);
    {   // the kernel addresses one batch row of a tensor with 32-bit byte offsets
        const int64_t widest = std::max<int64_t>(x_stride, std::max<int64_t>(di_, (int64_t)nheads * d_state));
        if ((int64_t)T * widest * 4 >= 0x7fffffffLL) return fail(MRS_E_SHAPE, "%s: one batch row of x, y, K or Q exceeds 2^31 bytes", fn);
    }
    if (dtype != MRS_F32 && dtype != MRS_F16 && dtype != MRS_BF16) return fail(MRS_E_DTYPE, "%s: dtype %d is not f32/f16/bf16", fn, dtype);
    if (!ssm_state || !k_state || !v_state || !y || !x || !K || !Q || !dt || !trap || !a_val || !D)
        return fail(MRS_E_NULL, "%s: null pointer", fn);
    if (batch < 1 || T < 1 || nheads < 1) return fail(MRS_E_SHAPE, "%s: batch=%d T=%d nheads=%d must be >= 1", fn, batch, T, nheads);
    if (chunk_size != kCS) return fail(MRS_E_SHAPE, "%s: chunk_size=%d, only %d is built", fn, chunk_size, kCS);
    if (!((headdim == 16 || headdim == 32 || headdim == 64) && (d_state == 16 || d_state == 32 || d_state == 64)))
        return fail(MRS_E_SHAPE, "%s: headdim=%d d_state=%d not in {16,32,64}x{16,32,64}", fn, headdim, d_state);
    if ((int64_t)batch * T * nheads * headdim > 0x7fffffffLL) return fail(MRS_E_SHAPE, "%s: batch*T*d_inner exceeds i32", fn);
    hipStream_t st = as_stream(stream);
    const int carry = (flags & MRS_M3_CARRY_STATE) ? 1 : 0;
    if (dtype == MRS_F32) {
        // f32 storage asks for 1e-4 parity, which 16-bit matrix-core operands cannot give:
        // run the recurrence itself (alpha/beta/gamma into the workspace, then the sequential kernel).
        const size_t n = (size_t)batch * T * nheads;
        if (!workspace || workspace_bytes < 3 * n * sizeof(float))
            return fail(MRS_E_WORKSPACE, "%s: f32 storage needs a workspace of %zu bytes", fn, 3 * n * sizeof(float));
        float *al = (float *)workspace, *be = al + n, *ga = be + n;
        int rc = mrs_m3_compute_abg(stream, al, be, ga, dt, a_val, trap, (int64_t)n);
        if (rc) return rc;
        if (!carry) {
            const int64_t ns = (int64_t)batch * nheads * headdim * d_state, nk = (int64_t)batch * nheads * d_state,
                          nv = (int64_t)batch * nheads * headdim;
            hipLaunchKernelGGL(zero_kernel, dim3((unsigned)((ns + 255) / 256)), dim3(256), 0, st, ssm_state, ns);
            hipLaunchKernelGGL(zero_kernel, dim3((unsigned)((nk + 255) / 256)), dim3(256), 0, st, k_state, nk);
            hipLaunchKernelGGL(zero_kernel, dim3((unsigned)((nv + 255) / 256)), dim3(256), 0, st, v_state, nv);
        }
        return mrs_m3_seq_fwd(stream, dtype, ssm_state, k_state, v_state, y, x, K, Q, al, be, ga, D, batch, T, nheads, headdim, d_state);
    }
    if (!aligned(x, 16) || !aligned(y, 16) || !aligned(K, 16) || !aligned(Q, 16) || !aligned(ssm_state, 16) || !aligned(k_state, 16))
        return fail(MRS_E_ALIGN, "%s: x, y, K, Q, ssm_state, k_state must be 16-byte aligned", fn);
    // Super-chunk split when the caller's workspace holds it; otherwise one workgroup walks the whole sequence.
    SsdSplit sp = {nullptr, nullptr, nullptr, 1, (T + kCS - 1) / kCS, x_stride, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, nullptr, 0};
    auto with_gen = [&](SsdSplit &o) {
        if (gen) { o.g_bn = gen->bn; o.g_cn = gen->cn; o.g_ang = gen->angle; o.g_bb = gen->b_bias; o.g_cb = gen->c_bias; o.g_bcs = gen->bc_stride; o.g_nr = gen->n_rope; o.g_head_major = gen->head_major; o.g_z = gen->gate; o.g_zs = gen->gate_stride; }
    };
    with_gen(sp);
    {
        int nsc, cps;
        ssd_plan(batch, T, nheads, nsc, cps);
        size_t o_dA, o_init;
        const size_t need = ssd_split_bytes(batch, nheads, headdim, d_state, nsc, &o_dA, &o_init);
        if (nsc > 1 && workspace && workspace_bytes >= need && aligned(workspace, 16)) {
            char *ws = (char *)workspace;
            sp = SsdSplit{(float *)ws, (float *)(ws + o_dA), (float *)(ws + o_init), nsc, cps, x_stride, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, nullptr, 0};
            with_gen(sp);
        }
    }
    if (dtype == MRS_BF16) return launch_ssd<bf16_t>(st, ssm_state, k_state, v_state, y, x, K, Q, dt, trap, a_val, D, sp, batch, T, nheads, headdim, d_state, carry);
    return launch_ssd<f16_t>(st, ssm_state, k_state, v_state, y, x, K, Q, dt, trap, a_val, D, sp, batch, T, nheads, headdim, d_state, carry);
}
