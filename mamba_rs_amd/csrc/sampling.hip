// Token sampling on the device: the reference's sample_token pipeline (src/module/sample.rs:243-265) --
// repetition penalty -> temperature -> top-k -> softmax -> top-p -> min-p -> weighted draw -- for every batch row in one
// launch, with the per-row xoshiro256++ generator (sample.rs:48-86) kept in device memory.  The reference downloads
// the logits and samples on the host (src/module/gpu_lm.rs:440-492); here a decode step needs no host round trip.
//
// One workgroup of 1024 threads owns a row (200 KB at a 50k vocabulary: it stays in L2 and is re-read with 16-byte
// loads).  Nothing is sorted: the k-th largest logit and the nucleus boundary are found by a 16-way search over the
// ordered bit patterns of the values -- 8 rounds of counting / mass sums; after the second round the few per cent of the
// row still inside the bracket are gathered into LDS and the remaining rounds walk that list -- and the filters become
// predicates on (value, index); the draw walks the kept weights in index order like weighted_sample does.  Sums are
// tree sums (f32 per lane, f64 across lanes) where the reference runs sequential f32 sums, so a draw within rounding
// distance of a boundary may land on the neighbouring token; among equal values the lower index is kept (the
// reference's select_nth_unstable / sort_unstable leave that open).
#include "common.hpp"

namespace mrs {

constexpr int kSampThreads = 1024;
constexpr int kSampWaves = kSampThreads / kWave;
constexpr int kListCap = 8192;   // bracket entries gathered into LDS
constexpr int kMaxBlocks = 1024; // block totals of the index-ordered walk
constexpr int kBinCopies = 32;   // copies of each histogram bin, one per lane modulo 32
constexpr int kFinish = 512;     // a bracket this small is resolved by ranking its entries against each other

struct SampShared {
    double d_slots[kSampWaves][16];
    double d_out[16];
    double blk[kMaxBlocks];
    float f_slots[kSampWaves];
    int idx_slots[kSampWaves];
    int found;
    float draw;
    int n_list;
    uint32_t list[kListCap];
    unsigned long long bins[16 * kBinCopies];
    unsigned long long hist[16];
    unsigned long long res_ge, res_gt;
    uint32_t res_key;
};

template <typename T> __device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
    return v;
}

// Wave total of a 32-bit value through the VALU's lane-crossing operand (no LDS traffic); the total is valid in lane 63
// only.  Pairs and quads by quad permutes, then the two mirrors inside a row of 16, then lane 15 of each row into the
// next row (rows 1 and 3), then lane 31 into rows 2 and 3.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ int dpp_mov(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ int wave_total_last(int v) {
    v += dpp_mov<0xB1, 0xf>(v);    // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E, 0xf>(v);    // quad_perm [2,3,0,1]
    v += dpp_mov<0x141, 0xf>(v);   // row_half_mirror
    v += dpp_mov<0x140, 0xf>(v);   // row_mirror
    v += dpp_mov<0x142, 0xa>(v);   // row_bcast:15 into rows 1, 3
    v += dpp_mov<0x143, 0xc>(v);   // row_bcast:31 into rows 2, 3
    return v;
}
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_movf(float v) {
    return __int_as_float(dpp_mov<CTRL, ROW_MASK>(__float_as_int(v)));   // masked-off rows receive the bit pattern 0 = +0.0f
}
__device__ __forceinline__ float wave_total_last(float v) {
    v += dpp_movf<0xB1, 0xf>(v);
    v += dpp_movf<0x4E, 0xf>(v);
    v += dpp_movf<0x141, 0xf>(v);
    v += dpp_movf<0x140, 0xf>(v);
    v += dpp_movf<0x142, 0xa>(v);
    v += dpp_movf<0x143, 0xc>(v);
    return v;
}

// Workgroup totals of v[0..N) left in sh.d_out[0..N) as f64 (int or float partials per lane and wave, f64 across waves).
template <int N, typename ACC> __device__ __forceinline__ void block_sum_to_lds(ACC (&v)[N], SampShared &sh) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < N; j++) v[j] = wave_total_last(v[j]);
    if (lane == 63) {
#pragma unroll
        for (int j = 0; j < N; j++) sh.d_slots[wave][j] = (double)v[j];
    }
    __syncthreads();
    if (threadIdx.x < N) {
        double s = 0.0;
        for (int w = 0; w < kSampWaves; w++) s += sh.d_slots[w][threadIdx.x];
        sh.d_out[threadIdx.x] = s;
    }
    __syncthreads();
}
__device__ __forceinline__ double block_sum1(float v, SampShared &sh) {
    float a[1] = {v};
    block_sum_to_lds(a, sh);
    return sh.d_out[0];
}

// Bit pattern whose unsigned order is the order of the floats (negative values flipped).
__device__ __forceinline__ uint32_t ordered_key(float x) {
    const uint32_t u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// One row in memory.  each(f) calls f(i, x) for this thread's share of the row, 4 consecutive entries per 16-byte load
// when the row allows it.
struct Row {
    const float *x;
    int vocab;
    bool vec;
    float scale;   // 1 / temperature, applied on the way in (1 when the stored row already carries it)
    __device__ __forceinline__ float at(int i) const { return x[i] * scale; }
    __device__ __forceinline__ float4 at4(int i0) const {
        float4 v = *reinterpret_cast<const float4 *>(x + i0);
        v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
        return v;
    }
    template <typename F> __device__ __forceinline__ void each(F f) const {
        if (vec) {
            const int n4 = vocab >> 2;
#pragma unroll 4
            for (int q = threadIdx.x; q < n4; q += kSampThreads) {
                const float4 v = at4(4 * q);
                f(4 * q, v.x); f(4 * q + 1, v.y); f(4 * q + 2, v.z); f(4 * q + 3, v.w);
            }
            for (int i = (n4 << 2) + threadIdx.x; i < vocab; i += kSampThreads) f(i, at(i));
        } else {
#pragma unroll 4
            for (int i = threadIdx.x; i < vocab; i += kSampThreads) f(i, at(i));
        }
    }
};

struct SearchOut { uint32_t key; unsigned long long ge, gt, thr; };

// Weight in 2^-32 units (saturating at 1): masses are summed as integers, so the totals do not depend on the order in
// which the lanes' additions land.
__device__ __forceinline__ unsigned long long fixed_weight(uint32_t weight_bits) {
    return (unsigned long long)__float2uint_rn(__uint_as_float(weight_bits) * 4294967296.0f);
}

// Largest key K such that the total over entries with key >= K still reaches the goal: at least `k` entries (MASS =
// false), or more than `p` of the whole mass (MASS = true; keys are then the bit patterns of non-negative weights).
// 8 rounds of a 16-way split of the bit range; a round is one histogram of the next 4 key bits over the entries still
// inside the bracket, built with LDS atomics on 32 copies of the 16 bins.  get(i, x, key) says whether an entry takes
// part and with which key.  Returns K, the totals over key >= K and key > K, and the goal in the same units.
template <bool MASS, typename Get> __device__ SearchOut search_key(const Row &row, Get get, int k, float p, SampShared &sh) {
    const int lane = threadIdx.x & 63;
    uint32_t lo = 0;
    unsigned long long above = 0, ge = 0, gt = 0, thr = MASS ? 0ull : (unsigned long long)k;
    bool listed = false;
    int n_list = 0;
    for (int shift = 28; shift >= 0; shift -= 4) {
        for (int t = threadIdx.x; t < 16 * kBinCopies; t += kSampThreads) sh.bins[t] = 0ull;
        __syncthreads();
        const bool whole = shift == 28;
        const uint32_t span = whole ? 0u : (16u << shift);   // the bracket is [lo, lo + span)
        auto tally = [&](uint32_t key) {
            if (key >= lo && (whole || key - lo < span)) {
                const uint32_t d = (key - lo) >> shift;
                atomicAdd(&sh.bins[d * kBinCopies + (lane & (kBinCopies - 1))], MASS ? fixed_weight(key) : 1ull);
            }
        };
        if (!listed) {
            row.each([&](int i, float x) {
                uint32_t key;
                if (get(i, x, key)) tally(key);
            });
        } else {
            for (int t = threadIdx.x; t < n_list; t += kSampThreads) tally(sh.list[t]);
        }
        __syncthreads();
        if (threadIdx.x < 16) {
            unsigned long long h = 0;
            for (int r = 0; r < kBinCopies; r++) h += sh.bins[threadIdx.x * kBinCopies + r];
            sh.hist[threadIdx.x] = h;
        }
        __syncthreads();
        if (MASS && whole) {   // the first round sees every entry: its total is the softmax denominator
            unsigned long long total = 0;
            for (int t = 0; t < 16; t++) total += sh.hist[t];
            thr = (unsigned long long)((double)p * (double)total);
        }
        // walk the bins from the top: the first one whose running total reaches the goal holds the answer
        unsigned long long run = 0, prev = 0;
        int jb = 0;
        ge = 0; gt = 0;
        bool found = false;
        for (int t = 15; t >= 0; t--) {
            prev = run;
            run += sh.hist[t];
            const bool holds = MASS ? above + run > thr : above + run >= thr;
            if (!found && (holds || t == 0)) { found = true; jb = t; ge = above + run; gt = above + prev; }
        }
        lo += (uint32_t)jb << shift;
        above = gt;
        if (!listed && shift > 0 && shift <= 24) {   // gather what is left inside the next bracket, if it fits
            if (threadIdx.x == 0) sh.n_list = 0;
            __syncthreads();
            const uint32_t nspan = 1u << shift;
            const uint32_t lo_now = lo;
            const int vocab = row.vocab;
            for (int i0 = 0; i0 < vocab; i0 += kSampThreads) {   // same trip count for all lanes: the ballots see whole waves
                const int i = i0 + (int)threadIdx.x;
                uint32_t key = 0;
                const bool in = i < vocab && get(i, row.at(i), key) && key >= lo_now && key - lo_now < nspan;
                const unsigned long long m = __ballot(in);
                if (m) {
                    const int leader = (int)__ffsll((long long)m) - 1;
                    int base = 0;
                    if (lane == leader) base = atomicAdd(&sh.n_list, (int)__popcll(m));
                    base = __shfl(base, leader, kWave);
                    const int slot = base + (int)__popcll(m & ((1ull << lane) - 1ull));
                    if (in && slot < kListCap) sh.list[slot] = key;
                }
            }
            __syncthreads();
            n_list = sh.n_list;
            listed = n_list <= kListCap;
            if (n_list <= kFinish) {
                // few enough to finish at once: every listed key totals what lies above it and what equals it; the key
                // whose "at or above" total reaches the goal while its "above" total does not is the answer
                if (threadIdx.x == 0) { sh.res_key = lo; sh.res_ge = ge; sh.res_gt = above; }
                __syncthreads();
                if ((int)threadIdx.x < n_list) {
                    const uint32_t mine = sh.list[threadIdx.x];
                    unsigned long long g = above, e = 0;
                    for (int u = 0; u < n_list; u++) {
                        const uint32_t ku = sh.list[u];
                        const unsigned long long c = MASS ? fixed_weight(ku) : 1ull;
                        g += ku > mine ? c : 0ull;
                        e += ku == mine ? c : 0ull;
                    }
                    const bool at = MASS ? g + e > thr : g + e >= thr, over = MASS ? g > thr : g >= thr;
                    if (at && !over) { sh.res_key = mine; sh.res_ge = g + e; sh.res_gt = g; }   // equal keys write equal values
                }
                __syncthreads();
                const SearchOut r{sh.res_key, sh.res_ge, sh.res_gt, thr};
                __syncthreads();
                return r;
            }
        }
    }
    return SearchOut{lo, ge, gt, thr};
}

// First index, in index order, whose inclusive running sum of w(i, x) exceeds `target`; vocab-1 when none does
// (weighted_sample's fall-through, sample.rs:239).  The row is cut into blocks of 256 entries (4 consecutive entries per
// lane); block totals go to LDS, one wave finds the block where the running sum crosses and then the entry inside it.
// With `relative` the target is that fraction of the total.
template <typename W> __device__ int ordered_find(const Row &row, W w, double target, bool relative, SampShared &sh) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int vocab = row.vocab;
    const int per = (vocab + 256 * kMaxBlocks - 1) / (256 * kMaxBlocks);   // 256-entry pieces per block: 1 up to 262144 entries
    const int bs = 256 * per;
    const int nb = (vocab + bs - 1) / bs;
    auto load4 = [&](int i0, float (&v)[4]) {   // weights of entries i0 .. i0+3 (0 past the end)
        if (row.vec && i0 + 3 < vocab) {
            const float4 q = row.at4(i0);
            v[0] = w(i0, q.x); v[1] = w(i0 + 1, q.y); v[2] = w(i0 + 2, q.z); v[3] = w(i0 + 3, q.w);
        } else {
#pragma unroll
            for (int c = 0; c < 4; c++) v[c] = i0 + c < vocab ? w(i0 + c, row.at(i0 + c)) : 0.0f;
        }
    };
#pragma unroll 2
    for (int b = wave; b < nb; b += kSampWaves) {
        float s = 0.0f;
        for (int sub = 0; sub < per; sub++) {
            float v[4];
            load4(b * bs + sub * 256 + lane * 4, v);
            s += (v[0] + v[1]) + (v[2] + v[3]);
        }
        s = wave_total_last(s);
        if (lane == 63) sh.blk[b] = (double)s;
    }
    if (threadIdx.x == 0) sh.found = vocab - 1;
    __syncthreads();
    if (wave == 0) {
        // running sum over the blocks: each lane a run of consecutive blocks, then a scan over the lanes
        const int chunk = (nb + kWave - 1) / kWave;
        const int b0 = lane * chunk;
        double mine = 0.0;
        for (int c = 0; c < chunk; c++) mine += b0 + c < nb ? sh.blk[b0 + c] : 0.0;
        double inc = mine;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const double t = __shfl_up(inc, d, kWave);
            if (lane >= d) inc += t;
        }
        if (relative) target *= __shfl(inc, kWave - 1, kWave);
        const unsigned long long hit = __ballot(inc > target);
        if (hit) {
            const int src = (int)__ffsll((long long)hit) - 1;
            // inside lane src's run of blocks
            double run = __shfl(inc - mine, src, kWave);
            const int sb0 = src * chunk;
            int blk = -1;
            for (int c = 0; c < chunk && blk < 0; c++) {
                const double t = sb0 + c < nb ? sh.blk[sb0 + c] : 0.0;
                if (run + t > target) blk = sb0 + c; else run += t;
            }
            if (blk < 0) blk = min(nb, sb0 + chunk) - 1;   // the lane total crossed, its partial sums rounded just below
            // inside the block
            int res = -1, last_pos = -1;
            for (int sub = 0; sub < per && res < 0; sub++) {
                const int i0 = blk * bs + sub * 256 + lane * 4;
                float v[4];
                load4(i0, v);
                const double lane_sum = ((double)v[0] + (double)v[1]) + ((double)v[2] + (double)v[3]);
                double li = lane_sum;
#pragma unroll
                for (int d = 1; d < kWave; d <<= 1) {
                    const double t = __shfl_up(li, d, kWave);
                    if (lane >= d) li += t;
                }
                const unsigned long long h2 = __ballot(run + li > target);
                double c = run + (li - lane_sum);
                int mine_idx = -1, mine_last = -1;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    c += (double)v[k];
                    if (mine_idx < 0 && c > target) mine_idx = i0 + k;
                    if (v[k] > 0.0f) mine_last = i0 + k;
                }
                if (h2) {
                    const int s2 = (int)__ffsll((long long)h2) - 1;
                    int cand = __shfl(mine_idx, s2, kWave);
                    const int cand_last = __shfl(mine_last, s2, kWave);
                    if (cand < 0) cand = cand_last;
                    res = cand;
                }
                const unsigned long long pos = __ballot(mine_last >= 0);
                if (pos) last_pos = __shfl(mine_last, 63 - (int)__clzll((long long)pos), kWave);
                run += __shfl(li, kWave - 1, kWave);
            }
            // the block total (f32 lane sums) said the crossing is here; if the running sums round just below it, the last
            // weighted entry of the block is the one
            if (lane == 0) sh.found = res >= 0 ? res : (last_pos >= 0 ? last_pos : vocab - 1);
        }
    }
    __syncthreads();
    const int r = sh.found;
    __syncthreads();
    return r;
}

__device__ __forceinline__ uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

// logits [rows, ld] f32 are read only; `work` [rows, ld] receives the penalised logits of rows with a penalty.  seen [rows, vocab] counts how often a token sits in the row's seen list (the penalty is applied once per
// occurrence, sample.rs:100-109).  rng [rows, 4] advances by one draw per sampled row (none on the greedy branch).
// Rows with active[row] == 0 are left alone.
__global__ __launch_bounds__(kSampThreads) void sample_rows_kernel(int *__restrict__ tokens, const float *__restrict__ logits,
                                                                   float *__restrict__ work, int64_t ld, int vocab,
                                                                   const mrs_sampler *__restrict__ samplers,
                                                                   const unsigned *__restrict__ seen,
                                                                   unsigned long long *__restrict__ rng,
                                                                   const int *__restrict__ active) {
    __shared__ SampShared sh;
    const int rowi = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (active && !active[rowi]) return;
    const mrs_sampler sp = samplers[rowi];
    const float *lrow = logits + (int64_t)rowi * ld;
    const float pen = sp.repetition_penalty;
    const bool pen_on = seen && isfinite(pen) && pen > 0.0f && pen != 1.0f;
    const bool greedy = sp.temperature <= 0.0f;
    const bool scale_on = !greedy && sp.temperature != 1.0f && sp.temperature > 0.0f;
    const float inv_t = scale_on ? 1.0f / sp.temperature : 1.0f;
    const bool vec = (ld % 4 == 0) && (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && (reinterpret_cast<uintptr_t>(work) % 16 == 0);

    // pass 1: penalty and temperature; maximum (and, for the greedy branch, the last index holding it)
    Row row{lrow, vocab, vec, 1.0f};
    float best = -INFINITY;
    int bi = 0;
    if (pen_on) {   // the penalised (and scaled) row goes to `work`; later passes read it from there
        float *wrow = work + (int64_t)rowi * ld;
        const unsigned *srow = seen + (int64_t)rowi * vocab;
        row.each([&](int i, float x) {
            for (unsigned c = srow[i]; c > 0; c--) x = x > 0.0f ? x / pen : x * pen;
            x *= inv_t;
            wrow[i] = x;
            if (x >= best) { best = x; bi = i; }   // a thread meets its entries in ascending index order
        });
        row.x = wrow;
        __syncthreads();   // the row is read back by other threads below (same workgroup, global memory)
    } else {
        row.scale = inv_t;   // temperature alone is applied on every read
        row.each([&](int i, float x) {
            if (x >= best) { best = x; bi = i; }
        });
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ov = __shfl_xor(best, m, kWave);
        const int oi = __shfl_xor(bi, m, kWave);
        if (ov > best || (ov == best && oi > bi)) { best = ov; bi = oi; }
    }
    if (lane == 0) { sh.f_slots[wave] = best; sh.idx_slots[wave] = bi; }
    __syncthreads();
    best = sh.f_slots[0]; bi = sh.idx_slots[0];
    for (int w = 1; w < kSampWaves; w++) {
        const float ov = sh.f_slots[w];
        const int oi = sh.idx_slots[w];
        if (ov > best || (ov == best && oi > bi)) { best = ov; bi = oi; }
    }
    if (greedy) {
        if (tid == 0) tokens[rowi] = bi;
        return;
    }
    const float xmax = best;

    // top-k: key of the k-th largest value, then how many entries equal to it stay (lowest indices first)
    const bool topk_on = sp.top_k > 0 && sp.top_k < vocab;
    uint32_t kkey = 0;       // keep_k(i) = key > kkey, or key == kkey and i <= k_tie_last
    int k_tie_last = vocab;
    if (topk_on) {
        const SearchOut r = search_key<false>(row, [](int, float x, uint32_t &key) { key = ordered_key(x); return true; }, sp.top_k, 0.0f, sh);
        kkey = r.key;
        const long long ties_kept = (long long)sp.top_k - (long long)r.gt, n_eq = (long long)(r.ge - r.gt);
        if (ties_kept < n_eq) {
            const uint32_t kk = kkey;
            k_tie_last = ordered_find(row, [=](int, float x) { return ordered_key(x) == kk ? 1.0f : 0.0f; }, (double)ties_kept - 0.5, false, sh);
        }
    }
    auto keep_k = [=](int i, float x) {
        if (!topk_on) return true;
        const uint32_t key = ordered_key(x);
        return key > kkey || (key == kkey && i <= k_tie_last);
    };
    // softmax weights e = exp(x - max) of the survivors
    auto weight = [=](float x) { return __expf(x - xmax); };

    // top-p: the largest weight value v whose mass of entries >= v still exceeds p * Z; entries above v stay, and as
    // many entries equal to v as it takes to cross p (sample.rs:170-204 on the descending order)
    const bool topp_on = isfinite(sp.top_p) && sp.top_p > 0.0f && sp.top_p < 1.0f;
    uint32_t pkey = 0;
    int p_tie_last = vocab;
    if (topp_on) {
        const SearchOut r = search_key<true>(
            row, [=](int i, float x, uint32_t &key) { if (!keep_k(i, x)) return false; key = __float_as_uint(weight(x)); return key != 0u; },
            0, sp.top_p, sh);
        pkey = r.key;
        const unsigned long long v = fixed_weight(pkey);
        if (pkey != 0 && v != 0) {
            // every entry equal to v adds exactly v: as many of them (lowest indices first) as it takes to cross
            const unsigned long long need = (r.thr >= r.gt ? (r.thr - r.gt) / v : 0ull) + 1ull, n_eq = (r.ge - r.gt) / v;
            if (need < n_eq) {
                const uint32_t pk = pkey;
                p_tie_last = ordered_find(row, [=](int i, float x) { return keep_k(i, x) && __float_as_uint(weight(x)) == pk ? 1.0f : 0.0f; },
                                          (double)need - 0.5, false, sh);
            }
        }
    }
    // min-p: entries below min_p x the largest probability go; the maximum's weight is exp(0) = 1
    const bool minp_on = sp.min_p > 0.0f;
    const float min_p = sp.min_p;
    auto final_weight = [=](int i, float x) -> float {
        if (!keep_k(i, x)) return 0.0f;
        const float e = weight(x);
        const uint32_t key = __float_as_uint(e);
        if (topp_on && !(key > pkey || (key == pkey && i <= p_tie_last))) return 0.0f;
        if (minp_on && e < min_p) return 0.0f;
        return e;
    };

    // the draw: one xoshiro256++ output per sampled token, mapped to [0, 1) by its top 24 bits
    if (tid == 0) {
        unsigned long long *s = rng + (int64_t)rowi * 4;
        uint64_t s0 = s[0], s1 = s[1], s2 = s[2], s3 = s[3];
        const uint64_t result = rotl64(s0 + s3, 23) + s0;
        const uint64_t t = s1 << 17;
        s2 ^= s0; s3 ^= s1; s1 ^= s2; s0 ^= s3; s2 ^= t; s3 = rotl64(s3, 45);
        s[0] = s0; s[1] = s1; s[2] = s2; s[3] = s3;
        sh.draw = (float)(result >> 40) / 16777216.0f;
    }
    __syncthreads();
    // first index whose running sum of kept weights exceeds draw x (their total)
    const int tok = ordered_find(row, final_weight, (double)sh.draw, true, sh);
    if (tid == 0) tokens[rowi] = tok;
}

int launch_sample_rows(hipStream_t st, int *tokens, const float *logits, float *work, int64_t ld, int rows, int vocab,
                       const mrs_sampler *samplers, const unsigned *seen, unsigned long long *rng, const int *active) {
    if (rows < 1 || vocab < 1 || ld < vocab) return fail(MRS_E_SHAPE, "sample: rows=%d vocab=%d ld=%lld", rows, vocab, (long long)ld);
    hipLaunchKernelGGL(sample_rows_kernel, dim3((unsigned)rows), dim3(kSampThreads), 0, st, tokens, logits, work, ld, vocab, samplers,
                       seen, rng, active);
    return check_launch("sample_rows_kernel");
}

}  // namespace mrs

extern "C" void mrs_xoshiro_seed(unsigned long long seed, unsigned long long state[4]) {
    uint64_t z = seed + 0x9E3779B97F4A7C15ull;
    for (int i = 0; i < 4; i++) {
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        state[i] = z ^ (z >> 31);
    }
    if (!state[0] && !state[1] && !state[2] && !state[3]) state[0] = 1;
}

extern "C" int mrs_sample_tokens(void *stream, int *tokens, const float *logits, float *work, int64_t ld, int rows, int vocab,
                                 const mrs_sampler *samplers, const unsigned *seen_counts, unsigned long long *rng_state,
                                 const int *active) {
    using namespace mrs;
    if (!tokens || !logits || !samplers || !rng_state) return fail(MRS_E_NULL, "mrs_sample_tokens: null pointer");
    if (seen_counts && !work) return fail(MRS_E_NULL, "mrs_sample_tokens: rows with a repetition penalty need the work buffer [rows, ld]");
    return launch_sample_rows(as_stream(stream), tokens, logits, work, ld, rows, vocab, samplers, seen_counts, rng_state, active);
}
