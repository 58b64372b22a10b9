"""GPU parity: the Mamba-1 backbone / LM engines vs the oracle's restatement of the reference CPU path.

The test bodies follow the reference's own engine tests (tests/m1_test_correctness.rs:17-146, 732-860;
tests/prefill.rs:173-232; tests/mixed_prefill_parity.rs:116-153).
"""
import numpy as np
import pytest

import orc
from util import cosine, det, max_rel, scaled_err

pytestmark = pytest.mark.gpu

from mamba_rs_amd import GpuMambaBackbone, GpuMambaLM, MambaConfig, MambaWeights, ScanMode, WeightDtype  # noqa: E402


def oracle_params(w: MambaWeights, cfg: MambaConfig, input_dim: int, round_to=None) -> orc.M1Params:
    """Copy product-side weights into the oracle's flat block (optionally with the bulk matrices rounded to a storage dtype)."""
    P = orc.M1Params(cfg.d_model, cfg.d_state, cfg.d_conv, cfg.expand, cfg.n_layers, max(input_dim, 1), seed=0)
    rq = (lambda a: orc.round_to(a, round_to)) if round_to is not None else (lambda a: a)
    if w.input_proj_w.size:
        P.input_proj_w[:] = w.input_proj_w; P.input_proj_b[:] = w.input_proj_b
    for l, lw in enumerate(w.layers):
        d = P.layers[l]
        d["norm_weight"][:] = lw.norm_weight
        d["in_proj_w"][:] = rq(lw.in_proj_w); d["x_proj_w"][:] = rq(lw.x_proj_w)
        d["dt_proj_w"][:] = rq(lw.dt_proj_w); d["out_proj_w"][:] = rq(lw.out_proj_w)
        d["conv1d_weight"][:] = lw.conv1d_weight; d["conv1d_bias"][:] = lw.conv1d_bias
        d["dt_proj_b"][:] = lw.dt_proj_b; d["a_log"][:] = lw.a_log; d["a_neg"][:] = -np.exp(lw.a_log); d["d_param"][:] = lw.d_param
    P.norm_f_weight[:] = w.norm_f_weight
    return P


TINY = MambaConfig(d_model=128, d_state=16, d_conv=4, expand=2, n_layers=2)   # the tiny CPU configuration


def test_weights_init_matches_oracle_init():
    w = MambaWeights.init(TINY, 128, 42)
    P = orc.M1Params(128, 16, 4, 2, 2, 128, seed=42)
    assert np.array_equal(w.input_proj_w, P.input_proj_w)
    for l in range(2):
        for k in ("in_proj_w", "conv1d_weight", "x_proj_w", "dt_proj_w", "out_proj_w"):
            assert np.array_equal(getattr(w.layers[l], k), P.layers[l][k]), k
        assert np.allclose(w.layers[l].dt_proj_b, P.layers[l]["dt_proj_b"], atol=2e-6)
        assert np.allclose(w.layers[l].a_log, P.layers[l]["a_log"], atol=2e-7)


def test_f32_engine_step_sequence_matches_cpu_reference_path():
    """Tiny config, f32, batch 1, 256 steps: every step output and the final states against the CPU route
    (tests/m1_test_correctness.rs:732-779 does this with max_diff < 5.0; here rel 1e-4 of the output scale)."""
    w = MambaWeights.init(TINY, 128, 42)
    P = oracle_params(w, TINY, 128)
    eng = GpuMambaBackbone.new(0, w, TINY, 128, 1)
    conv, ssm = orc.m1_zero_state(P)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((256, 128)).astype(np.float32)
    worst = 0.0
    for t in range(256):
        got = eng.step(x[t])
        want = orc.m1_backbone_step(P, x[t], conv, ssm)
        worst = max(worst, scaled_err(got[0], want))
    assert worst < 1e-4, worst
    for l in range(2):
        c, s = eng.download_state(l)
        assert scaled_err(s[0], ssm[l].reshape(256, 16)) < 1e-4
        assert np.allclose(c[0][:, 1:], conv[l].reshape(256, 3), atol=1e-5)       # GPU keeps d_conv slots, CPU d_conv-1
    # reset reproduces; state carries
    eng.reset()
    a = eng.step(x[0]); b = eng.step(x[0])
    assert np.max(np.abs(a - b)) > 1e-6
    eng.reset()
    assert np.array_equal(eng.step(x[0]), a)
    eng.close()


def test_f32_prefill_matches_cpu_prefill_and_hands_over_to_step():
    # tests/prefill.rs:173-232: prefill T then one step == T+1 steps (cos > 0.9999, max_rel < 1e-2)
    w = MambaWeights.init(TINY, 128, 42)
    P = oracle_params(w, TINY, 128)
    T = 256
    rng = np.random.default_rng(2)
    x = rng.standard_normal((T + 1, 128)).astype(np.float32)
    for mode in (ScanMode.SEQUENTIAL, ScanMode.PARALLEL):
        cfg = MambaConfig(d_model=128, d_state=16, d_conv=4, expand=2, n_layers=2, scan_mode=mode)
        eng = GpuMambaBackbone.new(0, w, cfg, 128, 1)
        last = eng.prefill_sequence(x[None, :T])
        conv, ssm = orc.m1_zero_state(P)
        ref = orc.m1_backbone_prefill(P, x[:T], conv, ssm)
        assert scaled_err(last[0], ref[-1]) < 1e-4, mode
        for l in range(2):
            assert scaled_err(eng.download_state(l)[1][0], ssm[l].reshape(256, 16)) < 1e-4
        nxt = eng.step(x[T])
        want = orc.m1_backbone_step(P, x[T], conv, ssm)
        assert cosine(nxt[0], want) > 0.9999 and max_rel(nxt[0], want, floor=1e-3) < 1e-2
        eng.close()


def test_batch_equals_individual_and_graph_equals_eager():
    # tests/m1_test_correctness.rs:100-146 (batch == individual) and :781-860 (graph == eager, 1e-5)
    cfg = MambaConfig(d_model=64, d_state=16, d_conv=4, expand=2, n_layers=3)
    w = MambaWeights.init(cfg, 20, 7)
    B = 4
    x = det(6 * B * 20, 9, 2.0).reshape(6, B, 20)
    eng = GpuMambaBackbone.new(0, w, cfg, 20, B)
    outs = [eng.step(x[t]) for t in range(6)]
    for b in range(B):
        one = GpuMambaBackbone.new(0, w, cfg, 20, 1)
        for t in range(6):
            assert np.allclose(one.step(x[t, b]), outs[t][b], atol=1e-5)
        one.close()
    eng.reset()
    eng.capture_graph()
    for t in range(6):
        assert np.allclose(eng.step(x[t]), outs[t], atol=1e-5), t      # replays stay equal to eager, step after step
    eng.reset()
    assert np.allclose(eng.step(x[0]), outs[0], atol=1e-5)
    eng.close()


@pytest.mark.parametrize("dtype", [WeightDtype.BF16, WeightDtype.F16])
def test_16bit_engine_tracks_f32_reference(dtype):
    """bf16/f16 storage engine vs the CPU route run on weights rounded to the storage type.  Activations are
    rounded between kernels, so this is a tolerance test: cosine >= 0.999 per step, as the reference's
    mixed-precision parity tests (tests/mixed_prefill_parity.rs:125-134)."""
    w = MambaWeights.init(TINY, 128, 42)
    code = orc.BF16 if dtype == WeightDtype.BF16 else orc.F16
    P = oracle_params(w, TINY, 128, round_to=code)
    eng = GpuMambaBackbone.new_with_dtype(0, w, TINY, 128, 2, dtype)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((40, 2, 128)).astype(np.float32)
    st = [orc.m1_zero_state(P) for _ in range(2)]
    for t in range(40):
        got = eng.step(x[t])
        for b in range(2):
            want = orc.m1_backbone_step(P, x[t, b], *st[b])
            assert cosine(got[b], want) >= 0.999, (t, b)
    # parallel-scan prefill route vs sequential route on the same engine type (mixed_prefill_parity.rs)
    T = 300
    xs = rng.standard_normal((2, T, 128)).astype(np.float32)
    outs = []
    for mode in (ScanMode.SEQUENTIAL, ScanMode.PARALLEL):
        cfg = MambaConfig(d_model=128, d_state=16, d_conv=4, expand=2, n_layers=2, scan_mode=mode)
        e2 = GpuMambaBackbone.new_with_dtype(0, w, cfg, 128, 2, dtype)
        outs.append((e2.prefill_sequence(xs), e2.download_state(1)[1]))
        e2.close()
    assert cosine(outs[0][0], outs[1][0]) >= 0.999 and cosine(outs[0][1], outs[1][1]) >= 0.999
    conv, ssm = orc.m1_zero_state(P)
    ref = orc.m1_backbone_prefill(P, xs[0], conv, ssm)
    assert cosine(outs[1][0][0], ref[-1]) >= 0.999
    eng.close()


def test_lm_greedy_decode_and_prefill():
    """Greedy LM loop with a tied head on a small random LM: every generated token must be the (last) argmax of
    the oracle's logits, for the step-by-step path and for prefill + decode."""
    cfg = MambaConfig(d_model=64, d_state=16, d_conv=4, expand=2, n_layers=2)
    w = MambaWeights.random_lm(cfg, seed=5, std=0.1)
    vocab = 300
    rng = np.random.default_rng(6)
    embed = (rng.standard_normal((vocab, 64)) * 0.5).astype(np.float32)
    P = oracle_params(w, cfg, 64)
    eng = GpuMambaBackbone.new(0, w, cfg, 64, 1)
    lm = GpuMambaLM(eng, embed)
    prompt = [int(v) for v in rng.integers(0, vocab, 12)]

    def oracle_generate(n):
        conv, ssm = orc.m1_zero_state(P)
        h = None
        for tok in prompt:
            h = orc.m1_backbone_step(P, embed[tok], conv, ssm, identity_proj=True)
        out = []
        for _ in range(n):
            logits = embed @ h
            tok = int(np.flatnonzero(logits == logits.max())[-1])
            margin = np.sort(logits)[-1] - np.sort(logits)[-2]
            out.append((tok, margin))
            h = orc.m1_backbone_step(P, embed[tok], conv, ssm, identity_proj=True)
        return out

    want = oracle_generate(8)
    got = lm.generate(prompt, 8)                          # prefill path
    for (tok, margin), g in zip(want, got):
        if margin < 1e-3:
            break                                          # a near-tie may legitimately flip across routes
        assert g == tok
    logits = lm.last_logits()
    assert logits.shape == (1, vocab) and np.isfinite(logits).all()
    # step-by-step path with a captured graph gives the same tokens as eager prefill path
    eng.reset()
    for tok in prompt[:-1]:
        lm.set_tokens([tok]); lm.decode_step()
    lm.set_tokens([prompt[-1]])
    lm.capture_graph()
    seq = []
    for _ in range(8):
        lm.decode_step(); seq.append(int(lm.get_tokens()[0]))
    assert seq[:3] == got[:3]
    lm.close(); eng.close()


def test_engine_rejects_bad_config():
    from mamba_rs_amd import MambaHipError
    cfg = MambaConfig(d_model=64, d_state=16, d_conv=4, expand=2, n_layers=1)
    w = MambaWeights.init(cfg, 10, 1)
    with pytest.raises(ValueError):
        GpuMambaBackbone.new(0, w, MambaConfig(d_model=64, d_state=300, n_layers=1), 10, 1)
    with pytest.raises(ValueError):
        GpuMambaBackbone.new(0, w, cfg, 11, 1)            # weight / input_dim mismatch
    eng = GpuMambaBackbone.new(0, w, cfg, 10, 1)
    with pytest.raises(ValueError):
        eng.step(np.zeros(3, np.float32))
    with pytest.raises(MambaHipError):
        eng.alloc_prefill_scratch(1)                      # one token is a step, not a prefill
    eng.alloc_prefill_scratch(16)
    eng.alloc_prefill_scratch(32)                         # the scratch follows the sequence length
    eng.close()


def test_16bit_engine_batch_above_64_takes_the_library_gemm_chain():
    """The own skinny GEMM serves batch <= 64; a batch of 65 runs add+RMSNorm, vendor GEMMs, conv step and the fused
    scan step instead.  Same bar as the small-batch chain: cosine >= 0.999 per step against the CPU route on rounded
    weights, and rows 0 and 64 (first row of the fifth 16-row tile, were it tiled) behave alike."""
    w = MambaWeights.init(TINY, 128, 43)
    P = oracle_params(w, TINY, 128, round_to=orc.BF16)
    B = 65
    eng = GpuMambaBackbone.new_with_dtype(0, w, TINY, 128, B, WeightDtype.BF16)
    rng = np.random.default_rng(8)
    x = rng.standard_normal((12, B, 128)).astype(np.float32)
    rows = (0, 31, 64)
    st = {b: orc.m1_zero_state(P) for b in rows}
    for t in range(12):
        got = eng.step(x[t])
        for b in rows:
            want = orc.m1_backbone_step(P, x[t, b], *st[b])
            assert cosine(got[b], want) >= 0.999, (t, b)
    eng.close()


def test_wide_dt_rank_at_large_batch_runs_dt_proj_as_its_own_gemm():
    """batch x dt_rank above the fusion limit (4096): the decode step takes delta from a GEMM instead of forming it
    inside the step kernel -- own-GEMM chain at batch 40, the last row count it takes for a wide model (d_model 2048 ->
    dt_rank 128, 40 x 128 = 5120), and library chain at batch 41 and 65."""
    cfg = MambaConfig(d_model=2048, d_state=16, d_conv=4, expand=1, n_layers=1)
    w = MambaWeights.init(cfg, 2048, 44)
    w.input_proj_w = np.zeros(0, np.float32); w.input_proj_b = np.zeros(0, np.float32)
    P = oracle_params(w, cfg, 2048, round_to=orc.BF16)
    P.input_proj_w[:] = np.eye(2048, dtype=np.float32); P.input_proj_b[:] = 0
    rng = np.random.default_rng(4)
    for B in (40, 41, 65):
        eng = GpuMambaBackbone.new_with_dtype(0, w, cfg, 2048, B, WeightDtype.BF16)
        x = rng.standard_normal((4, B, 2048)).astype(np.float32)
        rows = (0, B - 1)
        st = {b: orc.m1_zero_state(P) for b in rows}
        for t in range(4):
            got = eng.step(x[t])
            for b in rows:
                want = orc.m1_backbone_step(P, x[t, b], *st[b])
                assert cosine(got[b], want) >= 0.999, (B, t, b)
        eng.close()


@pytest.mark.parametrize("B", [100, 128])
def test_narrow_model_keeps_the_own_chain_up_to_128_rows(B):
    """Above 64 rows (up to 128 for narrow models) the decode chain still runs on the library's own GEMM, with dt_proj as
    a launch of its own (batch x dt_rank above the fusion limit).  First, middle and last row against the CPU route."""
    cfg = MambaConfig(d_model=768, d_state=16, d_conv=4, expand=2, n_layers=2)
    w = MambaWeights.random_lm(cfg, seed=B, std=0.05)
    P = oracle_params(w, cfg, 768, round_to=orc.BF16)
    P.input_proj_w[:] = np.eye(768, dtype=np.float32); P.input_proj_b[:] = 0
    rng = np.random.default_rng(B)
    eng = GpuMambaBackbone.new_with_dtype(0, w, cfg, 768, B, WeightDtype.BF16)
    x = rng.standard_normal((4, B, 768)).astype(np.float32)
    rows = (0, B // 2, B - 1)
    st = {b: orc.m1_zero_state(P) for b in rows}
    for t in range(4):
        if t == 2:
            eng.capture_graph()
        got = eng.step(x[t])
        for b in rows:
            want = orc.m1_backbone_step(P, x[t, b], *st[b])
            assert cosine(got[b], want) >= 0.999, (B, t, b)
    eng.close()


@pytest.mark.parametrize("B", [1, 3, 20])
def test_wide_model_runs_x_proj_as_a_split_k_launch(B):
    """d_inner 2048 x xdbl 96: a row's per-tile shares would be 48 KB, so x_proj does not ride in the in_proj launch; it
    runs as its own launch with K cut into slices whose shares the step kernel sums -- on the matrix cores also at one to
    four rows.  Checked against the CPU route on storage-rounded weights, step after step."""
    cfg = MambaConfig(d_model=1024, d_state=16, d_conv=4, expand=2, n_layers=2)
    w = MambaWeights.init(cfg, 1024, 45)
    w.input_proj_w = np.zeros(0, np.float32); w.input_proj_b = np.zeros(0, np.float32)
    P = oracle_params(w, cfg, 1024, round_to=orc.BF16)
    P.input_proj_w[:] = np.eye(1024, dtype=np.float32); P.input_proj_b[:] = 0
    rng = np.random.default_rng(B)
    eng = GpuMambaBackbone.new_with_dtype(0, w, cfg, 1024, B, WeightDtype.BF16)
    x = rng.standard_normal((5, B, 1024)).astype(np.float32)
    rows = sorted({0, B - 1})
    st = {b: orc.m1_zero_state(P) for b in rows}
    for t in range(5):
        if t == 2:
            eng.capture_graph()
        got = eng.step(x[t])
        for b in rows:
            want = orc.m1_backbone_step(P, x[t, b], *st[b])
            assert cosine(got[b], want) >= 0.999, (B, t, b)
    eng.close()


@pytest.mark.parametrize("dm,batch", [(256, 1), (256, 3), (512, 4), (768, 2), (768, 7), (256, 16), (512, 13)])
def test_few_row_decode_chain_with_folded_x_proj_equals_the_many_row_chain(dm, batch):
    """Up to 16 rows x_proj rides in the in_proj launch (per-tile shares, summed by the step kernel), and at one to four
    rows the projections take the lanes-along-the-row route; an engine of 24 rows runs x_proj as its own launch on the
    matrix cores.  Same weights, same inputs: the rows must agree to 16-bit rounding, step after step, eager and replayed."""
    cfg = MambaConfig(d_model=dm, d_state=16, d_conv=4, expand=2, n_layers=3)
    w = MambaWeights.random_lm(cfg, seed=dm + batch, std=0.05)
    few = GpuMambaBackbone.new_with_dtype(0, w, cfg, dm, batch, WeightDtype.BF16)
    many = GpuMambaBackbone.new_with_dtype(0, w, cfg, dm, 24, WeightDtype.BF16)
    rng = np.random.default_rng(dm)
    for t in range(24):
        if t == 8:
            few.capture_graph()
        x = rng.standard_normal((24, dm)).astype(np.float32)
        a, b = few.step(x[:batch]), many.step(x)[:batch]
        assert np.isfinite(a).all()
        assert cosine(a, b) >= 0.9995 and scaled_err(a, b) < 3e-2, (t, cosine(a, b), scaled_err(a, b))
    for layer in range(3):
        (ca, sa), (cb, sb) = few.download_state(layer), many.download_state(layer)
        assert cosine(sa, sb[:batch]) >= 0.9995 and cosine(ca, cb[:batch]) >= 0.9995
    few.close(); many.close()


def test_prefill_with_tuned_vendor_gemms_matches_the_default_choice_and_the_cpu_route():
    """set_gemm_tuning: the first prefill of 1024 rows or more times the GEMM library's kernels for each projection
    shape and later prefills run the fastest.  Another kernel sums in another order, so the tuned prefill is held to
    the untuned one by cosine and, like it, to the CPU route; tuned runs repeat bit for bit."""
    cfg = MambaConfig(d_model=256, d_state=16, d_conv=4, expand=2, n_layers=2)
    w = MambaWeights.init(cfg, 256, 77)
    P = oracle_params(w, cfg, 256, round_to=orc.BF16)
    B, T = 2, 512
    xs = (np.random.default_rng(5).standard_normal((B, T, 256)) * 0.5).astype(np.float32)
    eng = GpuMambaBackbone.new_with_dtype(0, w, cfg, 256, B, WeightDtype.BF16)
    print("case prefill, default vendor kernels", flush=True)
    base = eng.prefill_sequence(xs).copy()
    base_ssm = [eng.download_state(l)[1].copy() for l in range(2)]
    eng.set_gemm_tuning(True)
    runs = []
    for i in range(3):
        print(f"case prefill, tuned vendor kernels, run {i}", flush=True)
        eng.reset()
        runs.append((eng.prefill_sequence(xs).copy(), [eng.download_state(l)[1].copy() for l in range(2)]))
    for last, ssm in runs[1:]:
        assert np.array_equal(last, runs[0][0]) and all(np.array_equal(a, b) for a, b in zip(ssm, runs[0][1]))
    assert cosine(runs[0][0], base) >= 0.9999
    for l in range(2):
        assert cosine(runs[0][1][l], base_ssm[l]) >= 0.9999
    conv, ssm = orc.m1_zero_state(P)
    want = orc.m1_backbone_prefill(P, xs[1], conv, ssm)
    assert cosine(runs[0][0][1], want[-1]) >= 0.999
    eng.close()


@pytest.mark.parametrize("tuned", [False, True])
def test_decode_above_the_own_chain_limit_runs_the_projections_from_the_transposed_copies(tuned):
    """130 rows at d_model 768: past the own chain's limit, so in_proj and out_proj go to the GEMM library reading the
    transposed weight copies, x_proj and dt_proj reading the originals.  Eager steps, then replays of the captured step;
    with set_gemm_tuning the step that precedes the capture times the library's kernels for the four shapes and the
    graph holds the chosen ones.  First, middle and last row against the CPU route on storage-rounded weights."""
    B = 130
    cfg = MambaConfig(d_model=768, d_state=16, d_conv=4, expand=2, n_layers=2)
    w = MambaWeights.random_lm(cfg, seed=B, std=0.05)
    P = oracle_params(w, cfg, 768, round_to=orc.BF16)
    P.input_proj_w[:] = np.eye(768, dtype=np.float32); P.input_proj_b[:] = 0
    rng = np.random.default_rng(B)
    eng = GpuMambaBackbone.new_with_dtype(0, w, cfg, 768, B, WeightDtype.BF16)
    if tuned:
        eng.set_gemm_tuning(True)
    x = rng.standard_normal((5, B, 768)).astype(np.float32)
    rows = (0, B // 2, B - 1)
    st = {b: orc.m1_zero_state(P) for b in rows}
    for t in range(5):
        print(f"case library-chain decode, tuned={tuned}, step {t}", flush=True)
        if t == 2:
            eng.capture_graph()
        got = eng.step(x[t])
        for b in rows:
            want = orc.m1_backbone_step(P, x[t, b], *st[b])
            assert cosine(got[b], want) >= 0.999, (t, b)
    eng.close()


@pytest.mark.parametrize("shape", [
    # d_model, d_state, d_conv, expand, layers, input_dim, batch
    (128, 16, 4, 2, 3, 128, 1),      # the reference's default configuration
    (128, 16, 4, 2, 2, 128, 128),    # ... at the published batch size
    (64, 8, 2, 2, 2, 24, 5),         # input projection, short window, d_state 8
    (128, 64, 4, 2, 2, 128, 3),      # d_state 64: eight passes of the scan step
    (192, 16, 4, 1, 2, 192, 2),      # dt_rank 12: a second round of dt weights
    (128, 4, 3, 1, 4, 40, 7),        # expand 1, d_state 4 (one pass of 512 rows), dt_rank 8, x_proj row of 16
    (128, 16, 4, 2, 2, 130, 3),      # input row wider than d_model and not a multiple of four floats
    (64, 8, 4, 3, 2, 64, 2),         # expand 3
    (36, 16, 2, 3, 2, 36, 2),        # dt_rank 3: an x_proj row of 35 floats is outside the route, kernel chains on both sides
])
def test_small_f32_models_step_in_one_launch(shape, monkeypatch):
    """Small f32 engines (every product at most three rounds of sixteen weight rows per lane) run a backbone step as one kernel (one workgroup per batch row walks input
    projection, every layer and the final norm).  Held to the CPU route step after step (outputs 1e-4 of their scale, conv window
    and SSM state of every layer at the end), to the kernel chains it replaces (MRS_DECODE_NO_TINY=1 at creation), and
    to itself: graph replays and a second engine give the same bits."""
    dm, ds, dc, ex, L, idim, B = shape
    cfg = MambaConfig(d_model=dm, d_state=ds, d_conv=dc, expand=ex, n_layers=L)
    w = MambaWeights.init(cfg, idim, 7)
    P = oracle_params(w, cfg, idim)
    rng = np.random.default_rng(dm + B)
    steps = 6
    x = rng.standard_normal((steps, B, idim)).astype(np.float32)
    rows = sorted({0, B // 2, B - 1})
    st = {b: orc.m1_zero_state(P) for b in rows}
    print(f"case one-launch step {shape}", flush=True)
    eng = GpuMambaBackbone.new(0, w, cfg, idim, B)
    xd = cfg.dt_rank() + 2 * ds
    assert (eng.decode_route() == 2) == (xd % 4 == 0), (shape, eng.decode_route())   # 2 = the whole step in one launch
    assert eng.temporal_dtype() == WeightDtype.F32
    outs = []
    for t in range(steps):
        if t == 3:
            eng.capture_graph()
        got = eng.step(x[t])
        outs.append(got.copy())
        for b in rows:
            want = orc.m1_backbone_step(P, x[t, b], *st[b])
            assert scaled_err(got[b], want) < 1e-4, (t, b)
    for l in range(L):
        conv, ssm = eng.download_state(l)
        di = cfg.d_inner()
        for b in rows:
            # (the GPU keeps d_conv window slots, the CPU route d_conv - 1)
            assert np.allclose(conv[b][:, 1:], st[b][0][l].reshape(di, dc - 1), atol=1e-5), (l, b)
            assert scaled_err(ssm[b], st[b][1][l].reshape(di, ds)) < 1e-4, (l, b)
    eng.close()
    eng2 = GpuMambaBackbone.new(0, w, cfg, idim, B)
    for t in range(steps):
        assert np.array_equal(eng2.step(x[t]), outs[t]), t
    eng2.close()
    monkeypatch.setenv("MRS_DECODE_NO_TINY", "1")
    print(f"case kernel chains {shape}", flush=True)
    ref = GpuMambaBackbone.new(0, w, cfg, idim, B)
    assert ref.decode_route() != 2
    for t in range(steps):
        assert scaled_err(ref.step(x[t]), outs[t]) < 1e-4, t
    ref.close()
