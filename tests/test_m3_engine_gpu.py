"""GPU parity: the Mamba-3 SISO backbone engine (decode step) vs the oracle's restatement of the reference's CPU
layer (mamba3_layer_step, src/mamba3_siso/cpu/inference.rs:68-298), through the C ABI.

The bodies follow the reference's engine tests (tests/gpu_mamba3_lm_test.rs, tests/m3_cpu_gpu_train_parity.rs:
CPU route vs GPU route on the same weights, step by step, state compared at the end)."""
import numpy as np
import pytest

import orc
from util import cosine, scaled_err

pytestmark = pytest.mark.gpu

from mamba_rs_amd import GpuMamba3Backbone, Mamba3Config, Mamba3Weights, WeightDtype  # noqa: E402


def oracle_params(w: Mamba3Weights, cfg: Mamba3Config, input_dim: int, round_to=None) -> orc.M3Params:
    """Copy product-side weights into the oracle's flat block (bulk matrices optionally rounded to a storage type)."""
    P = orc.M3Params(cfg.d_model, cfg.d_state, cfg.expand, cfg.headdim, cfg.ngroups, cfg.n_layers, cfg.rope_fraction, input_dim,
                     seed=1, a_floor=cfg.a_floor, outproj_norm=cfg.is_outproj_norm)
    rq = (lambda a: orc.round_to(a, round_to)) if round_to is not None else (lambda a: a)
    P.input_proj_w[:] = w.input_proj_w; P.input_proj_b[:] = w.input_proj_b
    for l, lw in enumerate(w.layers):
        d = P.layers[l]
        for n in ("norm_weight", "dt_bias", "b_norm_weight", "c_norm_weight", "b_bias", "c_bias", "d_param", "norm_gate_weight"):
            d[n][:] = getattr(lw, n)
        d["in_proj_w"][:] = rq(lw.in_proj_w); d["out_proj_w"][:] = rq(lw.out_proj_w)
    P.norm_f_weight[:] = w.norm_f_weight
    return P


def perturbed(cfg, input_dim, seed):
    """init() leaves norms, biases and D at one; perturb them so that a dropped or swapped weight shows."""
    w = Mamba3Weights.init(cfg, input_dim, seed)
    rng = np.random.default_rng(seed + 7)
    for lw in w.layers:
        for n in ("norm_weight", "b_norm_weight", "c_norm_weight", "b_bias", "c_bias", "d_param", "norm_gate_weight"):
            a = getattr(lw, n)
            a += (rng.standard_normal(a.shape) * 0.2).astype(np.float32)
    w.norm_f_weight += (rng.standard_normal(w.norm_f_weight.shape) * 0.2).astype(np.float32)
    w.input_proj_b += (rng.standard_normal(w.input_proj_b.shape) * 0.1).astype(np.float32)
    return w


CONFIGS = [
    Mamba3Config(d_model=64, d_state=16, expand=2, headdim=16, ngroups=1, n_layers=2, rope_fraction=0.5),
    Mamba3Config(d_model=64, d_state=32, expand=2, headdim=32, ngroups=2, n_layers=2, rope_fraction=1.0, is_outproj_norm=True),
    Mamba3Config(d_model=64, d_state=64, expand=2, headdim=64, ngroups=1, n_layers=3, rope_fraction=0.5, a_floor=0.05),
]


@pytest.mark.parametrize("ci", range(len(CONFIGS)))
def test_f32_engine_steps_match_cpu_reference_path(ci):
    cfg = CONFIGS[ci]
    idim = 24
    w = perturbed(cfg, idim, 42 + ci)
    P = oracle_params(w, cfg, idim)
    eng = GpuMamba3Backbone.new(0, w, cfg, idim, 1)
    st = P.zero_state()
    rng = np.random.default_rng(ci)
    x = rng.standard_normal((96, idim)).astype(np.float32)
    print(f"case m3 engine f32 config={ci}", flush=True)
    worst = 0.0
    for t in range(96):
        got = eng.step(x[t])
        want = orc.m3_backbone_step(P, x[t], st)
        worst = max(worst, scaled_err(got[0], want))
    assert worst < 2e-4, worst
    L = cfg.n_layers - 1
    ssm, k, v, ang = eng.download_state(L)
    assert scaled_err(ssm[0], st[0][L]) < 2e-4 and scaled_err(k[0], st[1][L]) < 2e-4 and scaled_err(v[0], st[2][L]) < 2e-4
    if cfg.num_rope_angles():
        # angles live on a circle: compare through sin/cos
        assert np.max(np.abs(np.sin(ang[0]) - np.sin(st[3][L]))) < 1e-3 and np.max(np.abs(np.cos(ang[0]) - np.cos(st[3][L]))) < 1e-3
    eng.close()


@pytest.mark.parametrize("B", [1, 3])
def test_f32_engine_on_the_own_gemm_chain_matches_cpu_reference_path(B):
    """d_model and d_inner multiples of 128, one to four rows: the f32 engine takes the three-kernel layer (row-wise
    GEMM route on 4-byte operands) instead of the library chain; same bar as the library chain, eager and replayed."""
    cfg = Mamba3Config(d_model=128, d_state=32, expand=2, headdim=32, ngroups=1, n_layers=2, rope_fraction=0.5)
    w = perturbed(cfg, 40, 77)
    P = oracle_params(w, cfg, 40)
    eng = GpuMamba3Backbone.new(0, w, cfg, 40, B)
    st = [P.zero_state() for _ in range(B)]
    rng = np.random.default_rng(B)
    x = rng.standard_normal((48, B, 40)).astype(np.float32)
    worst = 0.0
    for t in range(48):
        if t == 16:
            eng.capture_graph()
        got = eng.step(x[t])
        for b in range(B):
            worst = max(worst, scaled_err(got[b], orc.m3_backbone_step(P, x[t, b], st[b])))
    assert worst < 2e-4, worst
    eng.close()


def test_batch_rows_are_independent_and_graph_equals_eager():
    cfg = CONFIGS[0]
    w = perturbed(cfg, 64, 5)
    w.input_proj_w = np.zeros(0, np.float32)   # identity projection (the LM case)
    rng = np.random.default_rng(9)
    x = rng.standard_normal((20, 3, 64)).astype(np.float32)
    for dtype in (WeightDtype.F32, WeightDtype.BF16):
        print(f"case m3 engine batch/graph dtype={dtype}", flush=True)
        eng = GpuMamba3Backbone.new_with_dtype(0, w, cfg, 64, 3, dtype)
        outs = np.stack([eng.step(x[t]) for t in range(20)])
        for b in range(3):
            solo = GpuMamba3Backbone.new_with_dtype(0, w, cfg, 64, 1, dtype)
            o1 = np.stack([solo.step(x[t, b]) for t in range(20)])
            assert np.allclose(o1[:, 0], outs[:, b], rtol=1e-5, atol=1e-5)
            solo.close()
        eng.reset()
        eng.capture_graph()
        outs_g = np.stack([eng.step(x[t]) for t in range(20)])
        assert np.array_equal(outs_g, outs)
        eng.close()


@pytest.mark.parametrize("dtype", [WeightDtype.BF16, WeightDtype.F16])
@pytest.mark.parametrize("ci,B", [(0, 2), (1, 2), (0, 7), (1, 21), (2, 16)])
def test_16bit_engine_tracks_cpu_path_on_rounded_weights(dtype, ci, B):
    """bf16/f16 storage (own-GEMM decode chain: folded RMSNorm, residual epilogue) vs the CPU route on weights
    rounded to the storage type: cosine >= 0.999 per step, the reference's mixed-precision bar.  From two rows up the
    projections run on the matrix cores and read tiled weights and tiled operands (2, 7 and 21 rows: one and two 16-row
    tiles, partly filled; 16: a whole one), eager for 24 steps, then replayed."""
    cfg = CONFIGS[ci]
    w = perturbed(cfg, 64, 11 + ci)
    w.input_proj_w = np.zeros(0, np.float32)
    code = orc.BF16 if dtype == WeightDtype.BF16 else orc.F16
    wi = Mamba3Weights(np.eye(64, dtype=np.float32), np.zeros(64, np.float32), w.layers, w.norm_f_weight)
    P = oracle_params(wi, cfg, 64, round_to=code)
    eng = GpuMamba3Backbone.new_with_dtype(0, w, cfg, 64, B, dtype)
    rows = sorted({0, B // 2, B - 1})
    st = {b: P.zero_state() for b in rows}
    rng = np.random.default_rng(3)
    x = rng.standard_normal((48, B, 64)).astype(np.float32)
    print(f"case m3 engine 16-bit dtype={dtype} config={ci} batch={B}", flush=True)
    for t in range(48):
        if t == 24:
            eng.capture_graph()
        got = eng.step(x[t])
        for b in rows:
            want = orc.m3_backbone_step(P, x[t, b], st[b])
            assert cosine(got[b], want) >= 0.999, (t, b)
    eng.close()


def test_create_rejects_bad_configs():
    from mamba_rs_amd import MambaHipError
    cfg = CONFIGS[0]
    w = Mamba3Weights.init(cfg, 16, 1)
    with pytest.raises(MambaHipError) as e:   # identity projection needs input_dim == d_model
        w2 = Mamba3Weights(np.zeros(0, np.float32), w.input_proj_b, w.layers, w.norm_f_weight)
        GpuMamba3Backbone.new(0, w2, cfg, 16, 1)
    assert e.value.code == -2
    with pytest.raises(ValueError):           # d_state 24 is not 4 x a power of two
        Mamba3Config(d_model=64, d_state=24, headdim=16).validate()


# ---- prefill ------------------------------------------------------------------------------------------

PREFILL_CASES = [(0, 150, WeightDtype.F32), (1, 97, WeightDtype.F32), (2, 130, WeightDtype.F32),
                 (0, 200, WeightDtype.BF16), (2, 200, WeightDtype.BF16), (1, 70, WeightDtype.F16), (2, 333, WeightDtype.F16)]


@pytest.mark.parametrize("ci,T,dtype", PREFILL_CASES)
def test_prefill_equals_T_steps_of_the_cpu_path_and_hands_off_to_step(ci, T, dtype):
    """Whole-sequence prefill (GEMMs over all rows, angle prefix sums, chunked SSD with carried state) against T
    single steps of the CPU layer: last-position output, final state of every kind, and the steps that follow
    (the handoff the reference tests in tests/prefill.rs:173-232 for Mamba-1)."""
    cfg = CONFIGS[ci]
    w = perturbed(cfg, 64, 21 + ci)
    w.input_proj_w = np.zeros(0, np.float32)
    wi = Mamba3Weights(np.eye(64, dtype=np.float32), np.zeros(64, np.float32), w.layers, w.norm_f_weight)
    code = {WeightDtype.F32: None, WeightDtype.BF16: orc.BF16, WeightDtype.F16: orc.F16}[dtype]
    P = oracle_params(wi, cfg, 64, round_to=code)
    B = 2
    rng = np.random.default_rng(31 + ci)
    xs = rng.standard_normal((B, T + 6, 64)).astype(np.float32)
    print(f"case m3 prefill config={ci} T={T} dtype={dtype}", flush=True)
    eng = GpuMamba3Backbone.new_with_dtype(0, w, cfg, 64, B, dtype)
    last = eng.prefill_sequence(xs[:, :T])
    st = [P.zero_state() for _ in range(B)]
    want_last = np.zeros((B, 64), np.float32)
    for b in range(B):
        for t in range(T):
            want_last[b] = orc.m3_backbone_step(P, xs[b, t], st[b])
    exact = dtype == WeightDtype.F32
    for b in range(B):
        if exact:
            assert scaled_err(last[b], want_last[b]) < 5e-4, (b, scaled_err(last[b], want_last[b]))
        else:
            assert cosine(last[b], want_last[b]) >= 0.999, (b, cosine(last[b], want_last[b]))
    L = cfg.n_layers - 1
    ssm, k, v, ang = eng.download_state(L)
    for b in range(B):
        tol_cos = 0.9999 if exact else 0.995
        assert cosine(ssm[b], st[b][0][L]) >= tol_cos and cosine(k[b], st[b][1][L]) >= tol_cos and cosine(v[b], st[b][2][L]) >= tol_cos
        if cfg.num_rope_angles():
            lim = 2e-3 if exact else 0.1
            assert np.max(np.abs(np.sin(ang[b]) - np.sin(st[b][3][L]))) < lim and np.max(np.abs(np.cos(ang[b]) - np.cos(st[b][3][L]))) < lim
    # handoff: the steps after the prefill continue the same trajectory
    for t in range(T, T + 6):
        got = eng.step(xs[:, t])
        for b in range(B):
            want = orc.m3_backbone_step(P, xs[b, t], st[b])
            if exact:
                assert scaled_err(got[b], want) < 5e-4, (t, b)
            else:
                assert cosine(got[b], want) >= 0.999, (t, b)
    eng.close()


def test_prefill_twice_continues_the_state_and_unsupported_chunk_shape_takes_the_sequential_route():
    """Two prefills of T steps == the CPU path over 2T steps (carried ssm/k/v/angle state); d_state 128 is outside the
    chunked kernel's shapes, so the engine forms alpha/beta/gamma and runs the recurrence kernel."""
    cfg = Mamba3Config(d_model=64, d_state=128, expand=2, headdim=16, ngroups=1, n_layers=2, rope_fraction=0.5)
    w = perturbed(cfg, 64, 77)
    w.input_proj_w = np.zeros(0, np.float32)
    wi = Mamba3Weights(np.eye(64, dtype=np.float32), np.zeros(64, np.float32), w.layers, w.norm_f_weight)
    P = oracle_params(wi, cfg, 64)
    T = 45
    rng = np.random.default_rng(5)
    xs = rng.standard_normal((1, 2 * T, 64)).astype(np.float32)
    eng = GpuMamba3Backbone.new(0, w, cfg, 64, 1)
    eng.prefill_sequence(xs[:, :T])
    last = eng.prefill_sequence(xs[:, T:])
    st = P.zero_state()
    for t in range(2 * T):
        want = orc.m3_backbone_step(P, xs[0, t], st)
    assert scaled_err(last[0], want) < 5e-4
    eng.close()


@pytest.mark.parametrize("dtype,T", [(WeightDtype.BF16, 1100), (WeightDtype.F16, 257)])
def test_scan_that_forms_K_and_Q_itself_equals_the_separate_K_Q_pass(dtype, T, monkeypatch):
    """headdim = d_state = 64, one group, 16-bit storage: the prefill's scan builds its K / Q tiles from the normalised
    B / C rows and the angles.  With MRS_M3_NO_FUSED_KQ set the engine writes K and Q with the separate kernel instead;
    both routes round the same K and Q to 16 bits (they differ by one fused multiply-add rounding in f32 before that), so
    the two prefills agree far inside the 16-bit bar: last output, every state, and the steps after the handoff.
    T covers the split into super-chunks (state-only pass) and a ragged last chunk."""
    cfg = CONFIGS[2]
    w = perturbed(cfg, 64, 91)
    w.input_proj_w = np.zeros(0, np.float32)
    B = 2
    rng = np.random.default_rng(17)
    xs = rng.standard_normal((B, T + 3, 64)).astype(np.float32)
    res = {}
    for route in ("fused", "separate"):
        if route == "separate":
            monkeypatch.setenv("MRS_M3_NO_FUSED_KQ", "1")
        else:
            monkeypatch.delenv("MRS_M3_NO_FUSED_KQ", raising=False)
        print(f"case m3 prefill K/Q route={route} T={T} dtype={dtype}", flush=True)
        eng = GpuMamba3Backbone.new_with_dtype(0, w, cfg, 64, B, dtype)
        last = eng.prefill_sequence(xs[:, :T]).copy()
        states = [eng.download_state(l) for l in range(cfg.n_layers)]
        after = np.stack([eng.step(xs[:, T + i]).copy() for i in range(3)])
        res[route] = (last, states, after)
        eng.close()
    fa, se = res["fused"], res["separate"]
    assert np.isfinite(fa[0]).all()
    assert scaled_err(fa[0], se[0]) < 1e-2 and cosine(fa[0].ravel(), se[0].ravel()) >= 0.9999
    assert scaled_err(fa[2], se[2]) < 1e-2
    # The first layer sees the same input on both routes: its states agree to the 16-bit rounding of K, and its angles
    # exactly.  The layers above integrate the small differences of their inputs over T steps in their angles (a sum
    # over time), which turns K and the state by that much: direction only.
    for a, b in zip(fa[1][0][:3], se[1][0][:3]):      # ssm, k, v
        assert scaled_err(a, b) < 1e-2
    assert np.array_equal(fa[1][0][3], se[1][0][3])
    for l in range(1, cfg.n_layers):
        for a, b in zip(fa[1][l][:3], se[1][l][:3]):
            assert cosine(a.ravel(), b.ravel()) >= 0.99, l
        assert np.max(np.abs(np.sin(fa[1][l][3]) - np.sin(se[1][l][3]))) < 0.2
    print("route difference: last", scaled_err(fa[0], se[0]), "layer-0 ssm", scaled_err(fa[1][0][0], se[1][0][0]),
          "top ssm", scaled_err(fa[1][-1][0], se[1][-1][0]), flush=True)


@pytest.mark.parametrize("case", [
    # config, input_dim, batch
    (Mamba3Config(d_model=128, d_state=16, expand=2, headdim=16, ngroups=1, n_layers=4, rope_fraction=0.5, a_floor=1e-4), 128, 1),   # the reference's default
    (Mamba3Config(d_model=128, d_state=16, expand=2, headdim=16, ngroups=1, n_layers=2, rope_fraction=0.5, a_floor=1e-4), 128, 128),
    (Mamba3Config(d_model=64, d_state=32, expand=2, headdim=32, ngroups=2, n_layers=2, rope_fraction=1.0, is_outproj_norm=True), 24, 5),
    (Mamba3Config(d_model=96, d_state=16, expand=2, headdim=16, ngroups=3, n_layers=3, rope_fraction=0.5), 40, 3),
    (Mamba3Config(d_model=128, d_state=16, expand=2, headdim=16, ngroups=1, n_layers=2, rope_fraction=0.5, a_floor=1e-4), 130, 3),   # input row wider than d_model, 2 mod 4
])
def test_small_f32_models_step_in_one_launch(case, monkeypatch):
    """f32 engines whose in_proj row is a multiple of four floats and fits in LDS run a backbone step as one kernel (one
    workgroup per batch row).  Held to the CPU route step after step (outputs and every state of the last layer), to the
    kernel chains it replaces (MRS_DECODE_NO_TINY=1 at creation), and to itself across graph replays and a second engine."""
    cfg, idim, B = case
    w = perturbed(cfg, idim, 11)
    P = oracle_params(w, cfg, idim)
    rng = np.random.default_rng(B + cfg.d_model)
    steps = 24
    x = rng.standard_normal((steps, B, idim)).astype(np.float32)
    rows = sorted({0, B // 2, B - 1})
    st = {b: P.zero_state() for b in rows}
    print(f"case m3 one-launch step d_model={cfg.d_model} batch={B}", flush=True)
    eng = GpuMamba3Backbone.new(0, w, cfg, idim, B)
    assert eng.decode_route() == 2, eng.decode_route()   # the whole step in one launch
    outs = []
    worst = 0.0
    for t in range(steps):
        if t == 8:
            eng.capture_graph()
        got = eng.step(x[t])
        outs.append(got.copy())
        for b in rows:
            worst = max(worst, scaled_err(got[b], orc.m3_backbone_step(P, x[t, b], st[b])))
    assert worst < 2e-4, worst
    L = cfg.n_layers - 1
    ssm, k, v, ang = eng.download_state(L)
    for b in rows:
        assert scaled_err(ssm[b], st[b][0][L]) < 2e-4 and scaled_err(k[b], st[b][1][L]) < 2e-4 and scaled_err(v[b], st[b][2][L]) < 2e-4, b
        if cfg.num_rope_angles():
            assert np.max(np.abs(np.sin(ang[b]) - np.sin(st[b][3][L]))) < 1e-3 and np.max(np.abs(np.cos(ang[b]) - np.cos(st[b][3][L]))) < 1e-3
    eng.close()
    eng2 = GpuMamba3Backbone.new(0, w, cfg, idim, B)
    for t in range(steps):
        assert np.array_equal(eng2.step(x[t]), outs[t]), t
    eng2.close()
    monkeypatch.setenv("MRS_DECODE_NO_TINY", "1")
    ref = GpuMamba3Backbone.new(0, w, cfg, idim, B)
    assert ref.decode_route() != 2
    for t in range(steps):
        assert scaled_err(ref.step(x[t]), outs[t]) < 2e-4, t
    ref.close()
