/*
 * sample_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the reference's token sampling (src/module/sample.rs) and of the
 * ragged-prompt generate_batch bookkeeping's building blocks: the xoshiro256++ generator,
 * repetition penalty, temperature, top-k, softmax (Cephes fast_exp, sequential f32 sums),
 * top-p, min-p and the weighted draw, in the reference's order of operations.
 *
 * Pins (tests/test_oracle_sample.py): the xoshiro256++ sequence from state {1,2,3,4} published
 * with the generator, SplitMix64's first output for seed 0, the reference's own unit tests
 * (sample.rs:267-389), and brute-force statements of each filter in numpy.
 *
 * Where the reference leaves the choice open (select_nth_unstable / sort_unstable among equal
 * values) this restatement keeps the lower index first.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

float orc_fast_exp(float x); /* mamba_oracle.c: fast_math.rs:54-74 */

/* ---- Xoshiro256PlusPlus, sample.rs:48-86 ------------------------------------------------ */
static inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

ORC_API void orc_xoshiro_seed(uint64_t seed, uint64_t s[4]) { /* sample.rs:54-66 */
    uint64_t z = seed + 0x9E3779B97F4A7C15ull;
    for (int i = 0; i < 4; i++) {
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        s[i] = z ^ (z >> 31);
    }
    if (!s[0] && !s[1] && !s[2] && !s[3]) s[0] = 1;
}

ORC_API uint64_t orc_xoshiro_next_u64(uint64_t s[4]) { /* sample.rs:68-81 */
    const uint64_t result = rotl64(s[0] + s[3], 23) + s[0];
    const uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return result;
}

ORC_API float orc_xoshiro_next_f32(uint64_t s[4]) { /* sample.rs:83-85 */
    return (float)(orc_xoshiro_next_u64(s) >> 40) / (float)(1ull << 24);
}

/* ---- filters ------------------------------------------------------------------------------ */
ORC_API void orc_apply_repetition_penalty(float *logits, int64_t n, const uint32_t *seen, int64_t n_seen, float penalty) { /* :93-110 */
    if (!isfinite(penalty) || penalty <= 0.0f || penalty == 1.0f) return;
    for (int64_t j = 0; j < n_seen; j++) {
        const int64_t idx = seen[j];
        if (idx < n) {
            if (logits[idx] > 0.0f) logits[idx] /= penalty;
            else logits[idx] *= penalty;
        }
    }
}

ORC_API void orc_apply_temperature(float *logits, int64_t n, float temperature) { /* :113-120 */
    if (temperature != 1.0f && temperature > 0.0f) {
        const float inv_t = 1.0f / temperature;
        for (int64_t i = 0; i < n; i++) logits[i] *= inv_t;
    }
}

typedef struct { float v; int64_t i; } vi_t;
static int cmp_desc(const void *a, const void *b) { /* descending by value, ascending by index among equals */
    const vi_t *x = (const vi_t *)a, *y = (const vi_t *)b;
    if (x->v > y->v) return -1;
    if (x->v < y->v) return 1;
    return (x->i > y->i) - (x->i < y->i);
}

ORC_API int64_t orc_apply_top_k(float *logits, int64_t n, int64_t k) { /* :124-144 */
    if (k == 0 || k >= n) return n;
    vi_t *a = (vi_t *)malloc((size_t)n * sizeof(vi_t));
    for (int64_t i = 0; i < n; i++) { a[i].v = logits[i]; a[i].i = i; }
    qsort(a, (size_t)n, sizeof(vi_t), cmp_desc);
    for (int64_t j = k; j < n; j++) logits[a[j].i] = -INFINITY;
    free(a);
    return k;
}

ORC_API void orc_softmax_inplace(float *logits, int64_t n) { /* :147-162 */
    float max = -INFINITY;
    for (int64_t i = 0; i < n; i++) max = fmaxf(max, logits[i]);
    for (int64_t i = 0; i < n; i++) logits[i] = orc_fast_exp(logits[i] - max);
    float sum = 0.0f;
    for (int64_t i = 0; i < n; i++) sum += logits[i];
    if (sum > 0.0f) {
        const float inv = 1.0f / sum;
        for (int64_t i = 0; i < n; i++) logits[i] *= inv;
    }
}

static void renormalize(float *p, int64_t n) { /* :219-227 */
    float sum = 0.0f;
    for (int64_t i = 0; i < n; i++) sum += p[i];
    if (sum > 0.0f && sum != 1.0f) {
        const float inv = 1.0f / sum;
        for (int64_t i = 0; i < n; i++) p[i] *= inv;
    }
}

ORC_API void orc_apply_top_p(float *probs, int64_t n, float p) { /* :170-204 */
    if (!isfinite(p) || p <= 0.0f || p >= 1.0f) return;
    vi_t *a = (vi_t *)malloc((size_t)(n > 0 ? n : 1) * sizeof(vi_t));
    int64_t m = 0;
    for (int64_t i = 0; i < n; i++)
        if (probs[i] > 0.0f) { a[m].v = probs[i]; a[m].i = i; m++; }
    qsort(a, (size_t)m, sizeof(vi_t), cmp_desc);
    float cumsum = 0.0f;
    int64_t cutoff = m;
    for (int64_t j = 0; j < m; j++) {
        cumsum += a[j].v;
        if (cumsum > p) { cutoff = j + 1; break; }
    }
    for (int64_t j = cutoff; j < m; j++) probs[a[j].i] = 0.0f;
    free(a);
    renormalize(probs, n);
}

ORC_API void orc_apply_min_p(float *probs, int64_t n, float min_p) { /* :207-217 */
    if (!(min_p > 0.0f)) return;      /* `min_p <= 0.0` returns; NaN falls through in the reference and then zeroes nothing */
    float maxp = 0.0f;
    for (int64_t i = 0; i < n; i++) maxp = fmaxf(maxp, probs[i]);
    const float thr = min_p * maxp;
    for (int64_t i = 0; i < n; i++)
        if (probs[i] < thr) probs[i] = 0.0f;
    renormalize(probs, n);
}

ORC_API uint32_t orc_weighted_sample(const float *probs, int64_t n, float r) { /* :230-240 with the draw passed in */
    float cumsum = 0.0f;
    for (int64_t i = 0; i < n; i++) {
        cumsum += probs[i];
        if (r < cumsum) return (uint32_t)i;
    }
    return (uint32_t)(n - 1);
}

/* sample_token, sample.rs:243-265.  `logits` is modified in place as in the reference (after the
 * call it holds the final probabilities, or the penalised logits on the greedy branch). */
ORC_API uint32_t orc_sample_token(float *logits, int64_t n, float temperature, int64_t top_k, float top_p, float min_p,
                                  float repetition_penalty, const uint32_t *seen, int64_t n_seen, uint64_t rng[4]) {
    orc_apply_repetition_penalty(logits, n, seen, n_seen, repetition_penalty);
    if (temperature <= 0.0f) { /* Iterator::max_by keeps the last maximum */
        int64_t best = 0;
        for (int64_t i = 1; i < n; i++)
            if (!(logits[i] < logits[best])) best = i;
        return (uint32_t)best;
    }
    orc_apply_temperature(logits, n, temperature);
    orc_apply_top_k(logits, n, top_k);
    orc_softmax_inplace(logits, n);
    orc_apply_top_p(logits, n, top_p);
    orc_apply_min_p(logits, n, min_p);
    return orc_weighted_sample(logits, n, orc_xoshiro_next_f32(rng));
}
