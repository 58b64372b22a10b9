"""GPU parity at the shapes the benchmark times: the 130m-shape LM (24 layers x d_model 768, vocab 50280, prefill
8 x 2048, decode at batch 64), the Mamba-3 backbone at 24 heads (prefill with K and Q formed in the scan, several
super-chunks, ragged tail, padded grid) and the 2.8b-shape layer (d_model 2560, dt_rank 160, xdbl 192).

Each engine runs at its real width through the C ABI and is held to the oracle's restatement of the reference's CPU
route on weights rounded to the storage type, on a few batch rows (rows are independent).  The engines round their
activations to 16 bits between kernels, the CPU route does not, so these are the reference's mixed-precision bars
(tests/mixed_prefill_parity.rs:125-134: cosine >= 0.999 on the last temporal and the SSM state; tests/prefill.rs:173-232
for the prefill -> step hand-off)."""
import numpy as np
import pytest

import orc
from util import cosine, scaled_err

pytestmark = pytest.mark.gpu

from mamba_rs_amd import (GpuMamba3Backbone, GpuMambaBackbone, GpuMambaLM, Mamba3Config, Mamba3Weights, MambaConfig,  # noqa: E402
                          MambaWeights, WeightDtype)
from test_engine_gpu import oracle_params  # noqa: E402
from test_m3_engine_gpu import oracle_params as m3_oracle_params, perturbed  # noqa: E402

COS = 0.999


def lm_oracle(cfg, w):
    P = oracle_params(w, cfg, cfg.d_model, round_to=orc.BF16)
    P.input_proj_w[:] = np.eye(cfg.d_model, dtype=np.float32); P.input_proj_b[:] = 0
    return P


def ssm_of(eng, layer, row):
    return eng.download_state(layer)[1][row]


# ---- 130m shape -------------------------------------------------------------------------------------------------------

CFG_130M = MambaConfig(d_model=768, d_state=16, d_conv=4, expand=2, n_layers=24)
VOCAB = 50280


@pytest.fixture(scope="module")
def lm130():
    w = MambaWeights.random_lm(CFG_130M, seed=130, std=0.02)
    rng = np.random.default_rng(131)
    embed = (rng.standard_normal((VOCAB, 768), dtype=np.float32) * np.float32(0.02))
    return w, embed, lm_oracle(CFG_130M, w), orc.round_to(embed, orc.BF16)


def test_130m_shape_decode_at_batch_64_follows_the_cpu_route(lm130):
    """24 layers, tied 50280-row head, 64 rows, graph replay from the third step on: rows 0, 31 and 63 against the CPU
    route step by step -- final-norm output (cosine), logits (cosine) and the greedy token, which must be the oracle's
    argmax whenever the oracle's lead over its runner-up exceeds four times the largest logit difference of the row."""
    w, embed, P, embed_r = lm130
    B, steps, rows = 64, 5, (0, 31, 63)
    print("case 130m-shape decode batch 64", flush=True)
    eng = GpuMambaBackbone.new_with_dtype(0, w, CFG_130M, 768, B, WeightDtype.BF16)
    lm = GpuMambaLM(eng, embed)
    rng = np.random.default_rng(7)
    toks = rng.integers(0, VOCAB, (steps, B)).astype(np.int32)
    st = {b: orc.m1_zero_state(P) for b in rows}
    compared = 0
    for t in range(steps):
        if t == 2:
            lm.capture_graph()
        lm.set_tokens(toks[t])
        lm.decode_step()
        logits = lm.last_logits()
        got_tok = lm.get_tokens()
        hid = eng.download_temporal()
        for b in rows:
            h = orc.m1_backbone_step(P, embed_r[toks[t, b]], *st[b], identity_proj=True)
            assert cosine(hid[b], h) >= COS, (t, b, cosine(hid[b], h))
            want = embed_r @ h
            assert cosine(logits[b], want) >= COS, (t, b)
            top2 = np.partition(want, -2)[-2:]
            if top2[1] - top2[0] > 4 * np.max(np.abs(logits[b] - want)):
                assert int(got_tok[b]) == int(np.flatnonzero(want == want.max())[-1]), (t, b)
                compared += 1
    for layer in (0, 23):
        for b in rows:
            s = ssm_of(eng, layer, b)
            ref = st[b][1][layer].reshape(1536, 16)
            assert cosine(s, ref) >= COS and scaled_err(s, ref) < 5e-2, (layer, b, cosine(s, ref), scaled_err(s, ref))
    print(f"greedy tokens compared: {compared} of {steps * len(rows)}", flush=True)
    lm.close(); eng.close()


def test_130m_shape_prefill_8x2048_follows_the_cpu_route_and_hands_off(lm130):
    """Prefill of 8 x 2048 embedded tokens (the T-split scan route, every layer) against the CPU prefill of rows 0 and 7:
    last-position output, final SSM state of the first and the last layer, then one decode step continuing from the
    prefilled state (tests/prefill.rs:173-232, tests/mixed_prefill_parity.rs:116-153)."""
    w, embed, P, embed_r = lm130
    B, T, rows = 8, 2048, (0, 7)
    print("case 130m-shape prefill 8 x 2048", flush=True)
    eng = GpuMambaBackbone.new_with_dtype(0, w, CFG_130M, 768, B, WeightDtype.BF16)
    rng = np.random.default_rng(8)
    toks = rng.integers(0, VOCAB, (B, T + 1))
    x = embed_r[toks]                                            # [B, T+1, 768] f32 on the bf16 grid
    last = eng.prefill_sequence(x[:, :T])
    states = {l: eng.download_state(l)[1] for l in (0, 23)}
    nxt = eng.step(x[:, T])
    for b in rows:
        conv, ssm = orc.m1_zero_state(P)
        ref = orc.m1_backbone_prefill(P, x[b, :T], conv, ssm, identity_proj=True)
        assert cosine(last[b], ref[-1]) >= COS, (b, cosine(last[b], ref[-1]))
        for l in (0, 23):
            r = ssm[l].reshape(1536, 16)
            assert cosine(states[l][b], r) >= COS and scaled_err(states[l][b], r) < 5e-2, (b, l, cosine(states[l][b], r))
        want = orc.m1_backbone_step(P, x[b, T], conv, ssm, identity_proj=True)
        assert cosine(nxt[b], want) >= COS, (b, cosine(nxt[b], want))
    eng.close()


def test_lm_generate_takes_any_sequence_of_prompt_lengths():
    """generate() prefills any prompt of two or more tokens, so one engine must serve prompts of different lengths one
    after the other (the reference allocates its prefill scratch per call, src/module/gpu_lm.rs:543-551); tokens are
    the oracle's argmax under the margin rule of the small-LM test.  Lengths 300 then 400 take the T-split scan, 3 then 7
    the serial one; generate_streaming goes through the same prefill for prompts of 256 tokens or more."""
    from mamba_rs_amd import SampleParams
    cfg = MambaConfig(d_model=64, d_state=16, d_conv=4, expand=2, n_layers=2)
    w = MambaWeights.random_lm(cfg, seed=5, std=0.1)
    vocab = 300
    rng = np.random.default_rng(6)
    embed = (rng.standard_normal((vocab, 64)) * 0.5).astype(np.float32)
    P = oracle_params(w, cfg, 64)
    P.input_proj_w[:] = np.eye(64, dtype=np.float32); P.input_proj_b[:] = 0
    eng = GpuMambaBackbone.new(0, w, cfg, 64, 1)
    lm = GpuMambaLM(eng, embed)

    def oracle_generate(prompt, n):
        conv, ssm = orc.m1_zero_state(P)
        for tok in prompt:
            h = orc.m1_backbone_step(P, embed[tok], conv, ssm, identity_proj=True)
        out = []
        for _ in range(n):
            logits = embed @ h
            tok = int(np.flatnonzero(logits == logits.max())[-1])
            srt = np.sort(logits)
            out.append((tok, srt[-1] - srt[-2]))
            h = orc.m1_backbone_step(P, embed[tok], conv, ssm, identity_proj=True)
        return out

    for n_prompt in (300, 400, 3, 7, 300):
        print(f"case generate prompt length {n_prompt}", flush=True)
        prompt = [int(v) for v in rng.integers(0, vocab, n_prompt)]
        want = oracle_generate(prompt, 6)
        got = lm.generate(prompt, 6)
        streamed = []
        lm.generate_streaming(prompt, SampleParams(temperature=0.0, max_tokens=6), lambda t: streamed.append(t) and False)
        for seq in (got, streamed):
            assert len(seq) == 6
            for (tok, margin), g in zip(want, seq):
                if margin < 1e-3:
                    break
                assert g == tok, (n_prompt, seq, [t for t, _ in want])
    lm.close(); eng.close()


# ---- 2.8b-shape layer ----------------------------------------------------------------------------------------------------

CFG_28B = MambaConfig(d_model=2560, d_state=16, d_conv=4, expand=2, n_layers=2)


@pytest.fixture(scope="module")
def w28():
    w = MambaWeights.random_lm(CFG_28B, seed=28, std=0.02)
    return w, lm_oracle(CFG_28B, w)


@pytest.mark.parametrize("B", [1, 2, 3, 5, 16, 23, 40, 64, 81, 128])
def test_28b_shape_decode_follows_the_cpu_route(w28, B):
    """d_model 2560 / d_inner 5120 / dt_rank 160 / xdbl 192, two layers: the row-wise route (1 row), the own chain on
    tiled weights and tiled activation operands at 3 to 64 rows -- one to four 16-row tiles, whole (16, 64) and partly
    filled (3, 5, 23, 40); x_proj split over K with the shares summed by the step kernel up to 25 rows, a dt_proj launch of
    its own above -- and the library chain (81 and 128 rows: x_proj split over K by the own GEMM and summed by a small
    kernel, the other projections by the GEMM library), eager then replayed."""
    w, P = w28
    print(f"case 2.8b-shape decode batch {B}", flush=True)
    assert CFG_28B.dt_rank() == 160 and CFG_28B.xdbl_dim() == 192
    eng = GpuMambaBackbone.new_with_dtype(0, w, CFG_28B, 2560, B, WeightDtype.BF16)
    assert eng.decode_route() == (0 if B > 64 else 1), eng.decode_route()   # 0: library chain, 1: own chain
    rng = np.random.default_rng(B)
    x = orc.round_to(rng.standard_normal((5, B, 2560)).astype(np.float32), orc.BF16)
    rows = sorted({0, B // 2, B - 1})
    st = {b: orc.m1_zero_state(P) for b in rows}
    for t in range(5):
        if t == 2:
            eng.capture_graph()
        got = eng.step(x[t])
        for b in rows:
            want = orc.m1_backbone_step(P, x[t, b], *st[b], identity_proj=True)
            assert cosine(got[b], want) >= COS, (t, b, cosine(got[b], want))
    for b in rows:
        s, r = ssm_of(eng, 1, b), st[b][1][1].reshape(5120, 16)
        assert cosine(s, r) >= COS and scaled_err(s, r) < 5e-2, (b, cosine(s, r), scaled_err(s, r))
    eng.close()


@pytest.mark.parametrize("T", [512, 4096])
def test_28b_shape_prefill_follows_the_cpu_route(w28, T):
    """4 x 512 and 4 x 4096 (the benchmarked prefill: a scan plan of nine chunks of 464 steps) through the 2.8b-shape
    layers (T-split scan at d_inner 5120 = 80 channel tiles, dt_proj with K = 160): rows 0 and 3 against the CPU
    prefill, then the hand-off step."""
    w, P = w28
    B = 4
    print(f"case 2.8b-shape prefill 4 x {T}", flush=True)
    eng = GpuMambaBackbone.new_with_dtype(0, w, CFG_28B, 2560, B, WeightDtype.BF16)
    rng = np.random.default_rng(29 + T)
    x = orc.round_to(rng.standard_normal((B, T + 1, 2560)).astype(np.float32), orc.BF16)
    last = eng.prefill_sequence(x[:, :T])
    state = eng.download_state(1)[1]
    nxt = eng.step(x[:, T])
    for b in (0, 3):
        print(f"  CPU route, row {b}", flush=True)
        conv, ssm = orc.m1_zero_state(P)
        ref = orc.m1_backbone_prefill(P, x[b, :T], conv, ssm, identity_proj=True)
        assert cosine(last[b], ref[-1]) >= COS, (b, cosine(last[b], ref[-1]))
        r = ssm[1].reshape(5120, 16)
        assert cosine(state[b], r) >= COS and scaled_err(state[b], r) < 5e-2, (b, cosine(state[b], r), scaled_err(state[b], r))
        want = orc.m1_backbone_step(P, x[b, T], conv, ssm, identity_proj=True)
        assert cosine(nxt[b], want) >= COS, (b, cosine(nxt[b], want))
    eng.close()


@pytest.mark.parametrize("d_model", [128, 1536, 2048, 4096])
def test_prefill_delta_kernel_at_every_dt_rank_width(d_model):
    """One layer, 2 x 80 steps (two and a half 64-row tiles: the last tile's spare lanes repeat the last row) at widths
    whose dt_rank is 8, 96, 128 and 256: the fused dt_proj + bias + softplus kernel of the 16-bit prefill with one, three,
    four and eight k-steps -- the weight in registers (64 columns per workgroup) and in LDS (128) -- against the CPU
    prefill: last output and final state.  (No hand-off step here: with a third of the channels at delta ~ 1e-5 and a
    seventh at delta ~ 25 the few large channels carry the output, and the decode chain's own rounding points -- f32
    x_proj shares where the prefill stores a 16-bit row -- show at 0.99 instead of 0.999; the hand-off is held to the
    CPU route at every width by the tests above, on weights as they come.)"""
    cfg = MambaConfig(d_model=d_model, d_state=16, d_conv=4, expand=2, n_layers=1)
    assert cfg.dt_rank() == {128: 8, 1536: 96, 2048: 128, 4096: 256}[d_model]
    w = MambaWeights.random_lm(cfg, seed=d_model, std=0.02)
    for lw in w.layers:      # a bias that reaches both sides of the softplus's small-argument branch and its pass-through
        lw.dt_proj_b[::3] -= 12.0
        lw.dt_proj_b[1::7] += 25.0
    P = lm_oracle(cfg, w)
    B, T = 2, 80
    print(f"case prefill delta kernel d_model={d_model}", flush=True)
    eng = GpuMambaBackbone.new_with_dtype(0, w, cfg, d_model, B, WeightDtype.BF16)
    rng = np.random.default_rng(d_model)
    x = orc.round_to(rng.standard_normal((B, T, d_model)).astype(np.float32), orc.BF16)
    last = eng.prefill_sequence(x)
    state = eng.download_state(0)[1]
    for b in range(B):
        conv, ssm = orc.m1_zero_state(P)
        ref = orc.m1_backbone_prefill(P, x[b], conv, ssm, identity_proj=True)
        assert cosine(last[b], ref[-1]) >= COS, (b, cosine(last[b], ref[-1]))
        r = ssm[0].reshape(2 * d_model, 16)
        assert cosine(state[b], r) >= COS and scaled_err(state[b], r) < 5e-2, (b, cosine(state[b], r), scaled_err(state[b], r))
    eng.close()


# ---- Mamba-3 backbone at 24 heads -----------------------------------------------------------------------------------

CFG_M3 = Mamba3Config(d_model=768, d_state=64, expand=2, headdim=64, ngroups=1, n_layers=2, rope_fraction=0.5)


@pytest.fixture(scope="module")
def m3w():
    w = perturbed(CFG_M3, 768, 303)
    w.input_proj_w = np.zeros(0, np.float32)
    wi = Mamba3Weights(np.eye(768, dtype=np.float32), np.zeros(768, np.float32), w.layers, w.norm_f_weight)
    return w, m3_oracle_params(wi, CFG_M3, 768, round_to=orc.BF16)


def test_m3_24_heads_prefill_with_K_and_Q_formed_in_the_scan_follows_the_cpu_route(m3w):
    """d_model 768 -> 24 heads x 64 x 64, batch 3, T = 1100: nine super-chunks of two chunks, a 12-step tail and a grid
    padded from 27 to 32 groups -- the workgroup -> (row, head, super-chunk) mapping of the route that forms K and Q in
    the scan, held to T single steps of the CPU layer on rows 0 and 2: last output, ssm / k / v state and angles of both
    layers, then the hand-off steps."""
    w, P = m3w
    B, T = 3, 1100
    assert CFG_M3.nheads() == 24
    print("case m3 24-head prefill fused K/Q vs cpu route", flush=True)
    rng = np.random.default_rng(33)
    xs = rng.standard_normal((B, T + 3, 768)).astype(np.float32)
    eng = GpuMamba3Backbone.new_with_dtype(0, w, CFG_M3, 768, B, WeightDtype.BF16)
    last = eng.prefill_sequence(xs[:, :T])
    states = [eng.download_state(l) for l in range(2)]
    after = [eng.step(xs[:, T + i]).copy() for i in range(3)]
    for b in (0, 2):
        st = P.zero_state()
        for t in range(T):
            want = orc.m3_backbone_step(P, xs[b, t], st)
        assert cosine(last[b], want) >= COS, (b, cosine(last[b], want))
        for l in range(2):
            ssm, k, v, ang = states[l]
            for name, got, ref in (("ssm", ssm[b], st[0][l]), ("k", k[b], st[1][l]), ("v", v[b], st[2][l])):
                # per head as well: a head mapped to another head's rows would hide in the whole-tensor cosine
                for h in range(24):
                    assert cosine(got[h], ref[h]) >= 0.995, (b, l, name, h, cosine(got[h], ref[h]))
            # Angles are running sums over the 1100 steps.  The first layer sees the oracle's input exactly; the second
            # integrates the 16-bit rounding of its input rows step after step (measured: 0.17 at the worst pair).
            lim = 0.1 if l == 0 else 0.35
            da = max(np.max(np.abs(np.sin(ang[b]) - np.sin(st[3][l]))), np.max(np.abs(np.cos(ang[b]) - np.cos(st[3][l]))))
            assert da < lim, (b, l, float(da))
        for i in range(3):
            want = orc.m3_backbone_step(P, xs[b, T + i], st)
            assert cosine(after[i][b], want) >= COS, (b, i, cosine(after[i][b], want))
    eng.close()


def test_m3_24_heads_4x4096_both_K_Q_routes_agree(m3w, monkeypatch):
    """The benchmark's prefill shape, batch 4 x 4096 at 24 heads: the scan that forms K and Q itself against the route
    that reads them from memory (whose kernel is held to the f64 chunked oracle at this size in test_m3_gpu.py)."""
    w, _ = m3w
    B, T = 4, 4096
    rng = np.random.default_rng(34)
    xs = rng.standard_normal((B, T, 768)).astype(np.float32)
    res = {}
    for route in ("fused", "separate"):
        if route == "separate":
            monkeypatch.setenv("MRS_M3_NO_FUSED_KQ", "1")
        else:
            monkeypatch.delenv("MRS_M3_NO_FUSED_KQ", raising=False)
        print(f"case m3 24-head 4x4096 route={route}", flush=True)
        eng = GpuMamba3Backbone.new_with_dtype(0, w, CFG_M3, 768, B, WeightDtype.BF16)
        last = eng.prefill_sequence(xs).copy()
        res[route] = (last, eng.download_state(0), eng.download_state(1))
        eng.close()
    fa, se = res["fused"], res["separate"]
    assert np.isfinite(fa[0]).all()
    assert cosine(fa[0].ravel(), se[0].ravel()) >= 0.9999 and scaled_err(fa[0], se[0]) < 2e-2
    for a, b in zip(fa[1][:3], se[1][:3]):            # first layer: same input on both routes
        assert scaled_err(a, b) < 1e-2
        for bi in range(B):
            for h in range(24):
                assert cosine(a[bi, h], b[bi, h]) >= 0.9999, (bi, h)
    assert np.array_equal(fa[1][3], se[1][3])
    for a, b in zip(fa[2][:3], se[2][:3]):
        assert cosine(a.ravel(), b.ravel()) >= 0.99
