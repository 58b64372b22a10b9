"""Pins for the sampling part of the CPU oracle (oracle/sample_oracle.c). CPU only.

Known answers: the xoshiro256++ outputs from state {1, 2, 3, 4} published with the generator (the rand_xoshiro test
vector), SplitMix64's first output for seed 0, the reference's unit tests (src/module/sample.rs:267-389) and numpy
statements of each filter on random inputs.
"""
import numpy as np

import orc

M64 = (1 << 64) - 1


def test_xoshiro256pp_known_sequence():
    rng = orc.Xoshiro(state=[1, 2, 3, 4])
    want = [41943041, 58720359, 3588806011781223, 3591011842654386, 9228616714210784205, 9973669472204895162,
            14011001112246962877, 12406186145184390807, 15849039046786891736, 10450023813501588000]
    assert [rng.next_u64() for _ in range(10)] == want


def test_xoshiro_python_restatement_agrees_on_a_long_run():
    """An independent pure-Python statement of the generator and of the seeding chain (sample.rs:54-81)."""
    def seed_state(seed):
        z, s = (seed + 0x9E3779B97F4A7C15) & M64, []
        for _ in range(4):
            z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
            z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
            s.append(z ^ (z >> 31))
        return s

    rotl = lambda x, k: ((x << k) | (x >> (64 - k))) & M64
    for seed in (0, 42, 99, M64):
        s = seed_state(seed)
        rng = orc.Xoshiro(seed=seed)
        assert rng.state() == s
        for _ in range(200):
            out = (rotl((s[0] + s[3]) & M64, 23) + s[0]) & M64
            t = (s[1] << 17) & M64
            s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3]; s[2] ^= t; s[3] = rotl(s[3], 45)
            assert rng.next_u64() == out
    # first slot for seed 0 is SplitMix64's first output for seed 0
    assert orc.Xoshiro(seed=0).state()[0] == 0xE220A8397B1DCDAF
    r = orc.Xoshiro(seed=42)
    ref = orc.Xoshiro(seed=42)
    for _ in range(100):
        f = r.next_f32()
        assert f == (ref.next_u64() >> 40) / float(1 << 24) and 0.0 <= f < 1.0


def test_reference_unit_tests():
    rng = orc.Xoshiro(seed=42)
    assert orc.sample_token([1.0, 5.0, 2.0, 0.5], rng, temperature=0.0)[0] == 1                    # test_greedy_argmax
    t = orc.apply_temperature([2.0, 1.0, 0.0, -1.0], 2.0)                                          # test_temperature_scaling
    assert abs(t[0] - 1.0) < 1e-6 and abs(t[1] - 0.5) < 1e-6
    for _ in range(100):                                                                           # test_topk_k1_is_argmax
        assert orc.sample_token([1.0, 5.0, 2.0, 0.5], rng, temperature=1.0, top_k=1)[0] == 1
    seen = set()
    for _ in range(1000):                                                                          # test_topk_k2_excludes_rest
        seen.add(orc.sample_token([1.0, 5.0, 3.0, 0.1], rng, temperature=1.0, top_k=2)[0])
    assert seen == {1, 2}
    p = orc.apply_top_p([0.6, 0.3, 0.05, 0.05], 0.85)                                              # test_topp_filters_tail
    assert (p[2] == 0.0 or p[3] == 0.0) and p[0] > 0 and p[1] > 0
    p = orc.apply_min_p([0.5, 0.3, 0.1, 0.05, 0.05], 0.2)                                          # test_minp_filters_by_fraction
    assert p[0] > 0 and p[1] > 0 and p[3] == 0 and p[4] == 0
    assert abs(orc.apply_repetition_penalty([2.0, -1.0, 0.0], [0], 2.0)[0] - 1.0) < 1e-6           # ..._positive_divides
    assert abs(orc.apply_repetition_penalty([2.0, -1.0, 0.0], [1], 2.0)[1] + 2.0) < 1e-6           # ..._negative_multiplies
    logits = [1.0, 2.0, 1.5, 0.8, 3.0, 0.1, 0.5, 2.5]
    def run(seed, n):
        g = orc.Xoshiro(seed=seed)
        return [orc.sample_token(logits, g, temperature=0.8)[0] for _ in range(n)]
    assert run(42, 20) == run(42, 20)                                                              # test_deterministic_with_seed
    assert run(42, 50) != run(99, 50)                                                              # test_different_seed_...


def test_filters_against_numpy_statements():
    rng = np.random.default_rng(0)
    for trial in range(20):
        n = int(rng.integers(5, 400))
        x = (rng.standard_normal(n) * 3).astype(np.float32)
        # repetition penalty: applied once per occurrence; disabled for 1.0, <= 0 and NaN
        seen = rng.integers(0, n + 3, 12)
        want = x.copy()
        for t in seen:
            if t < n:
                want[t] = want[t] / np.float32(1.3) if want[t] > 0 else want[t] * np.float32(1.3)
        assert (orc.apply_repetition_penalty(x, seen, 1.3) == want).all()
        for off in (1.0, 0.0, -2.0, float("nan")):
            assert (orc.apply_repetition_penalty(x, seen, off) == x).all()
        # temperature: multiply by the f32 reciprocal; disabled for 1.0 and <= 0
        assert (orc.apply_temperature(x, 0.7) == x * (np.float32(1.0) / np.float32(0.7))).all()
        assert (orc.apply_temperature(x, 1.0) == x).all() and (orc.apply_temperature(x, -1.0) == x).all()
        # top-k keeps exactly the k largest
        k = int(rng.integers(1, n))
        tk = orc.apply_top_k(x, k)
        kept = np.isfinite(tk)
        assert kept.sum() == k and (tk[kept] == x[kept]).all() and x[kept].min() >= x[~kept].max()
        assert (orc.apply_top_k(x, 0) == x).all() and (orc.apply_top_k(x, n) == x).all()
        # softmax: sums to one, ratios follow exp
        p = orc.softmax(tk)
        e = np.exp(x.astype(np.float64) - x.max()) * kept
        assert abs(p.sum() - 1.0) < 1e-5 and np.allclose(p, e / e.sum(), rtol=2e-6, atol=1e-30) and (p[~kept] == 0).all()
        # top-p: the smallest descending prefix whose mass exceeds p, renormalised
        pp = float(rng.uniform(0.05, 0.98))
        order = np.argsort(-p.astype(np.float64), kind="stable")
        cs = np.cumsum(p[order].astype(np.float32), dtype=np.float32)
        cut = int(np.argmax(cs > np.float32(pp))) + 1 if (cs > np.float32(pp)).any() else n
        keep = np.zeros(n, bool); keep[order[:cut]] = True; keep &= p > 0
        tp = orc.apply_top_p(p, pp)
        assert ((tp > 0) == keep).all() and abs(tp.sum() - 1.0) < 1e-5
        assert np.allclose(tp[keep] / tp[keep].sum(), p[keep] / p[keep].sum(), rtol=1e-5)
        for off in (1.0, 1.5, 0.0, -0.1, float("nan")):
            assert (orc.apply_top_p(p, off) == p).all()
        # min-p: drop entries below min_p x the maximum, renormalise
        mp = orc.apply_min_p(p, 0.1)
        keep = p >= np.float32(0.1) * p.max()
        assert ((mp > 0) == (keep & (p > 0))).all() and abs(mp.sum() - 1.0) < 1e-5
        assert (orc.apply_min_p(p, 0.0) == p).all()
        # weighted draw: first index whose running f32 sum exceeds r; the last index when none does
        r = float(rng.uniform())
        cs = np.cumsum(p, dtype=np.float32)
        want_i = int(np.argmax(np.float32(r) < cs)) if (np.float32(r) < cs).any() else n - 1
        assert orc.weighted_sample(p, r) == want_i
        assert orc.weighted_sample(np.zeros(n, np.float32), 0.5) == n - 1


def test_sample_token_is_the_composition_and_consumes_one_draw():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(300) * 2).astype(np.float32)
    g1, g2 = orc.Xoshiro(seed=7), orc.Xoshiro(seed=7)
    for _ in range(30):
        tok, _ = orc.sample_token(x, g1, temperature=0.9, top_k=40, top_p=0.9, min_p=0.05, repetition_penalty=1.2, seen=[3, 3, 10])
        p = orc.apply_min_p(orc.apply_top_p(orc.softmax(orc.apply_top_k(orc.apply_temperature(
            orc.apply_repetition_penalty(x, [3, 3, 10], 1.2), 0.9), 40)), 0.9), 0.05)
        assert tok == orc.weighted_sample(p, g2.next_f32())
    assert g1.state() == g2.state()
    # the greedy branch draws nothing and keeps the last maximum
    g = orc.Xoshiro(seed=1); s0 = g.state()
    assert orc.sample_token([1.0, 4.0, 4.0, 0.0], g, temperature=0.0)[0] == 2 and g.state() == s0
    # empirical frequencies follow the softmax
    g = orc.Xoshiro(seed=11)
    logits = np.array([0.0, 1.0, 2.0, -1.0], np.float32)
    counts = np.bincount([orc.sample_token(logits, g)[0] for _ in range(20000)], minlength=4) / 20000.0
    assert np.abs(counts - np.exp(logits) / np.exp(logits).sum()).max() < 0.012
