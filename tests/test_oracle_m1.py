"""Pins for the Mamba-1 part of the CPU oracle (oracle/mamba_oracle.c).

The reference holds no golden vectors for this path (its tests are relational),
so each oracle function is pinned by (a) the reference's own relational tests
re-expressed here, (b) closed forms / library routines, (c) independent
brute-force restatements in numpy on small inputs.  CPU only.
"""
import math

import numpy as np
import pytest
import torch

import orc
from util import cosine, det, max_rel, scaled_err, scan_inputs


# ---------------------------------------------------------------- rounding --
def test_round_bf16_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 20000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, -3.3895314e38, np.inf, -np.inf, 1e-40, 65504.0],
                 dtype=np.float32),
    ])
    got = orc.round_to(x, orc.BF16)
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert math.isnan(orc.lib().orc_round_bf16(float("nan")))


def test_round_bf16_ties_to_even():
    # 1 + 2^-8 is exactly halfway between bf16 neighbours 1.0 and 1+2^-7 -> even (1.0);
    # 1 + 3*2^-8 is halfway between 1+2^-7 and 1+2^-6 -> even (1+2^-6)
    assert orc.lib().orc_round_bf16(1.0 + 2.0 ** -8) == 1.0
    assert orc.lib().orc_round_bf16(1.0 + 3 * 2.0 ** -8) == 1.0 + 2.0 ** -6


def test_round_f16_matches_numpy():
    rng = np.random.default_rng(2)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 6.1e-5, np.inf, -np.inf], dtype=np.float32),
    ])
    got = orc.round_to(x, orc.F16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ---------------------------------------------------------------- fast_exp --
def test_fast_exp_accuracy_bounds():
    # src/ops/fast_math.rs:277-294 and :325-340: max relative error < 2e-7
    xs = np.arange(-800, 201, dtype=np.float32) * np.float32(0.1)
    got = orc.fast_exp(xs).astype(np.float64)
    exact = np.exp(xs.astype(np.float64))
    keep = exact > 1e-30
    assert np.max(np.abs(got[keep] - exact[keep]) / exact[keep]) < 2e-7
    xs = -np.arange(1000, dtype=np.float32) * np.float32(0.08)
    got = orc.fast_exp(xs).astype(np.float64)
    exact = np.exp(xs.astype(np.float64))
    keep = exact > 1e-30
    assert np.max(np.abs(got[keep] - exact[keep]) / exact[keep]) < 2e-7


def test_fast_exp_edge_cases():
    # src/ops/fast_math.rs:313-323
    fe = orc.lib().orc_fast_exp
    assert fe(-100.0) >= 0.0 and math.isfinite(fe(-100.0)) and math.isfinite(fe(100.0))
    assert abs(fe(0.0) - 1.0) < 1e-8
    assert abs(fe(-0.5) - math.exp(-0.5)) < 1e-7
    assert abs(fe(-1.0) - math.exp(-1.0)) < 1e-7


def test_activations_are_library_routines():
    xs = np.linspace(-30, 30, 601, dtype=np.float32)
    L = orc.lib()
    for x in xs:
        xd = float(x)
        sp = math.log1p(math.exp(xd)) if xd <= 20 else xd
        si = xd / (1.0 + math.exp(-xd))
        for f in (L.orc_cpu_softplus, L.orc_gpu_softplus):
            assert abs(f(xd) - sp) <= 2e-6 * max(1.0, abs(sp))
        for f in (L.orc_cpu_silu, L.orc_gpu_silu):
            assert abs(f(xd) - si) <= 2e-6 * max(1.0, abs(si))
    # threshold: above 20 softplus passes its argument through unchanged
    assert L.orc_cpu_softplus(20.5) == 20.5 and L.orc_gpu_softplus(25.0) == 25.0


# ----------------------------------------------------------- scan dispatch --
def test_scan_use_parallel_reference_values():
    # tests/scan_mode_boundary.rs:12-53
    SEQ, PAR, AUTO = 0, 1, 2
    THR = 256
    assert not orc.scan_use_parallel(AUTO, THR - 1, 16)
    assert not orc.scan_use_parallel(AUTO, THR, 16)
    assert orc.scan_use_parallel(AUTO, THR + 1, 16)
    for mode in (SEQ, PAR, AUTO):
        assert orc.scan_use_parallel(mode, 1, 65)
    assert not orc.scan_use_parallel(SEQ, 1 << 20, 16)
    assert orc.scan_use_parallel(PAR, 1, 16)


# ------------------------------------------------------------------- scan ---
def _direct_scan(h0, delta, u, Bm, Cm, a_neg, D):
    """Non-recurrent closed form in float64 numpy:
    h_t[n] = exp(a_n S_t) h_0[n] + sum_{s<=t} exp(a_n (S_t - S_s)) delta_s u_s B_s[n],  S = cumsum(delta)."""
    batch, T, di = delta.shape
    ds = a_neg.shape[1]
    y = np.zeros((batch, T, di))
    hT = np.zeros((batch, di, ds))
    for b in range(batch):
        for d in range(di):
            S = np.cumsum(delta[b, :, d].astype(np.float64))
            a = a_neg[d].astype(np.float64)
            du = delta[b, :, d].astype(np.float64) * u[b, :, d].astype(np.float64)
            for t in range(T):
                w = np.exp(np.outer(S[t] - S[: t + 1], a))            # [t+1, ds]
                ht = np.exp(a * S[t]) * h0[b, d] + (w * du[: t + 1, None] * Bm[b, : t + 1].astype(np.float64)).sum(0)
                y[b, t, d] = ht @ Cm[b, t].astype(np.float64) + float(D[d]) * float(u[b, t, d])
            hT[b, d] = ht
    return y, hT


def test_scan_f64_vs_direct_closed_form():
    rng = np.random.default_rng(3)
    inp = scan_inputs(rng, 2, 9, 5, 4, s4d=False)
    h0 = rng.standard_normal((2, 5, 4)) * 0.3
    y, h = orc.m1_scan_f64(h0, inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"])
    yd, hd = _direct_scan(h0, inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"])
    assert np.max(np.abs(y - yd)) < 1e-12 and np.max(np.abs(h - hd)) < 1e-12


def test_scan_special_cases():
    rng = np.random.default_rng(4)
    inp = scan_inputs(rng, 1, 6, 3, 4)
    h0 = rng.standard_normal((1, 3, 4))
    # delta = 0: state unchanged, y = C.h + D u
    z = np.zeros_like(inp["delta"])
    y, h = orc.m1_scan_f64(h0, z, inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"])
    assert np.array_equal(h, h0)
    want = np.einsum("bdn,btn->btd", h0, inp["C"].astype(np.float64)) + inp["D"] * inp["u"].astype(np.float64)
    assert np.allclose(y, want, atol=1e-13)
    # B = 0: h_T = prod_t exp(delta_t a) h_0 = exp(a * sum delta) h_0
    y, h = orc.m1_scan_f64(h0, inp["delta"], inp["u"], np.zeros_like(inp["B"]), inp["C"], inp["a_neg"], inp["D"])
    S = inp["delta"].astype(np.float64).sum(1)                      # [B, di]
    assert np.allclose(h, np.exp(S[:, :, None] * inp["a_neg"][None]) * h0, rtol=1e-12)
    # constant inputs, h0 = 0: geometric series h_T = du B (1 - r^T)/(1 - r), r = exp(delta a)
    T, dl, uu = 7, 0.25, -1.5
    delta = np.full((1, T, 1), dl, np.float32); u = np.full((1, T, 1), uu, np.float32)
    Bm = np.full((1, T, 2), 0.5, np.float32); Cm = np.ones((1, T, 2), np.float32)
    a = np.array([[-1.0, -3.0]], np.float32); D = np.array([2.0], np.float32)
    y, h = orc.m1_scan_f64(np.zeros((1, 1, 2)), delta, u, Bm, Cm, a, D)
    r = np.exp(dl * a[0].astype(np.float64))
    hT = dl * uu * 0.5 * (1 - r ** T) / (1 - r)
    assert np.allclose(h[0, 0], hT, rtol=1e-12)
    assert np.isclose(y[0, -1, 0], hT.sum() + 2.0 * uu, rtol=1e-12)


def test_scan_chunking_and_gate_modes():
    rng = np.random.default_rng(5)
    inp = scan_inputs(rng, 2, 20, 6, 8, s4d=False)
    h0 = rng.standard_normal((2, 6, 8)) * 0.1
    a = (inp["delta"], inp["u"], inp["B"], inp["C"])
    y, h = orc.m1_scan_f64(h0, *a, inp["a_neg"], inp["D"])
    y1, h1 = orc.m1_scan_f64(h0, *[t[:, :13] for t in a], inp["a_neg"], inp["D"])
    y2, h2 = orc.m1_scan_f64(h1, *[t[:, 13:] for t in a], inp["a_neg"], inp["D"])
    assert np.array_equal(np.concatenate([y1, y2], 1), y) and np.array_equal(h2, h)   # state carry is exact
    z = inp["z"]
    silu = z.astype(np.float64) / (1 + np.exp(-z.astype(np.float64)))
    yg2, _ = orc.m1_scan_f64(h0, *a, inp["a_neg"], inp["D"], gate=z, gate_mode=2)
    assert np.allclose(yg2, y * silu, rtol=1e-13)
    yg1, _ = orc.m1_scan_f64(h0, *a, inp["a_neg"], inp["D"], gate=z, gate_mode=1)
    assert np.allclose(yg1, y * z.astype(np.float64), rtol=1e-13)


@pytest.mark.parametrize("s4d", [True, False])
def test_scan_f32_routes_track_ground_truth(s4d):
    rng = np.random.default_rng(6)
    inp = scan_inputs(rng, 2, 300, 16, 16, s4d=s4d)
    h0 = (rng.standard_normal((2, 16, 16)) * 0.1).astype(np.float32)
    a = (inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"])
    y, h = orc.m1_scan_f64(h0, *a, gate=inp["z"], gate_mode=2)
    for route in (orc.m1_scan_cpu, orc.m1_scan_gpu):
        yr, hr = route(h0, *a, gate=inp["z"], gate_mode=2)
        assert scaled_err(yr, y) < 2e-6 and scaled_err(hr, h) < 2e-6
    # bf16 storage of y on the GPU route costs at most half a bf16 ulp (2^-9) per element
    yb, _ = orc.m1_scan_gpu(h0, *a, gate=inp["z"], gate_mode=2, dtype=orc.BF16)
    assert max_rel(yb, y, floor=1e-3) < 2.0 ** -8


def test_scan_cpu_route_threads_bitwise():
    # Parallel == Single bitwise: channels are independent (tests/prefill.rs:136-168)
    rng = np.random.default_rng(7)
    inp = scan_inputs(rng, 2, 64, 40, 16)
    h0 = np.zeros((2, 40, 16), np.float32)
    a = (inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"])
    y1, h1 = orc.m1_scan_cpu(h0, *a, threads=1)
    y8, h8 = orc.m1_scan_cpu(h0, *a, threads=8)
    assert np.array_equal(y1, y8) and np.array_equal(h1, h8)


def test_scan_strided_bc_equals_gathered():
    rng = np.random.default_rng(8)
    inp = scan_inputs(rng, 1, 10, 4, 4)
    xd = 3 + 2 * 4
    xdbl = rng.standard_normal((1, 10, xd)).astype(np.float32)
    Bv, Cv = xdbl[:, :, 3:7], xdbl[:, :, 7:11]
    h0 = np.zeros((1, 4, 4))
    y_ref, _ = orc.m1_scan_f64(h0, inp["delta"], inp["u"], Bv.copy(), Cv.copy(), inp["a_neg"], inp["D"])
    # strided call straight into xdbl
    import ctypes
    L = orc.lib()
    h = np.zeros((1, 4, 4)); y = np.zeros((1, 10, 4))
    base = xdbl.ctypes.data
    L.orc_m1_scan_f64(orc._p(h), orc._p(y), orc._p(inp["delta"]), orc._p(inp["u"]), ctypes.c_void_p(base + 4 * 3),
                      ctypes.c_void_p(base + 4 * 7), ctypes.c_int64(xd), orc._p(inp["a_neg"]), orc._p(inp["D"]), None,
                      ctypes.c_int(0), ctypes.c_int64(1), ctypes.c_int64(10), ctypes.c_int64(4), ctypes.c_int64(4))
    assert np.array_equal(y, y_ref)


# ------------------------------------------------------------------ conv1d --
def _torch_conv_silu(x, w, bias, hist):
    """x [B,T,di], hist [B,di,dc-1] (inputs before t=0, oldest first) -> silu(conv), f64."""
    xt = torch.from_numpy(np.concatenate([np.transpose(hist, (0, 2, 1)), x], axis=1)).double().transpose(1, 2)
    wt = torch.from_numpy(w).double().unsqueeze(1)
    out = torch.nn.functional.conv1d(xt, wt, torch.from_numpy(bias).double(), groups=w.shape[0])
    return torch.nn.functional.silu(out).transpose(1, 2).numpy()


@pytest.mark.parametrize("dc", [2, 3, 4, 8])
def test_conv1d_f64_is_depthwise_causal_conv(dc):
    rng = np.random.default_rng(10 + dc)
    B, T, di = 2, 11, 5
    x = rng.standard_normal((B, T, di)).astype(np.float32)
    w = rng.standard_normal((di, dc)).astype(np.float32)
    bias = rng.standard_normal(di).astype(np.float32)
    st0 = rng.standard_normal((B, di, dc)).astype(np.float32)
    out, st = orc.conv1d_seq_f64(st0, x, w, bias)
    want = _torch_conv_silu(x, w, bias, st0[:, :, 1:])
    assert np.allclose(out, want, atol=1e-12)
    # window after the call = last dc inputs of (old window ++ x)
    full = np.concatenate([np.transpose(st0, (0, 2, 1)), x], axis=1)
    assert np.array_equal(st, np.transpose(full[:, -dc:], (0, 2, 1)))
    # carried history: two calls == one call over the concatenation
    o1, s1 = orc.conv1d_seq_f64(st0, x[:, :4], w, bias)
    o2, s2 = orc.conv1d_seq_f64(s1, x[:, 4:], w, bias)
    assert np.array_equal(np.concatenate([o1, o2], 1), out) and np.array_equal(s2, st)
    # T shorter than the window keeps the older slots
    o3, s3 = orc.conv1d_seq_f64(st0, x[:, :1], w, bias)
    assert np.array_equal(s3[:, :, :-1], st0[:, :, 1:].astype(np.float64))


def test_conv1d_routes_agree():
    rng = np.random.default_rng(20)
    T, di, dc = 9, 6, 4
    x = rng.standard_normal((1, T, di)).astype(np.float32)
    w = rng.standard_normal((di, dc)).astype(np.float32)
    bias = rng.standard_normal(di).astype(np.float32)
    out, _ = orc.conv1d_seq_f64(np.zeros((1, di, dc)), x, w, bias)
    og, _ = orc.conv1d_seq_gpu(np.zeros((1, di, dc)), x, w, bias)
    assert scaled_err(og, out) < 1e-6
    hist = np.zeros((di, dc - 1), np.float32)
    for t in range(T):  # CPU route keeps dc-1 history, "dot before shift" (cpu/inference.rs:119-139)
        ut, hist = orc.conv1d_step_cpu(x[0, t], hist, w, bias)
        assert scaled_err(ut, out[0, t]) < 1e-6
    assert np.array_equal(hist, x[0, -(dc - 1):].T)


# -------------------------------------------------------------- weight init --
_A, _C, _M = 6364136223846793005, 1442695040888963407, 1 << 64


def _lcg_draw(seed, k):
    """k-th draw (1-based) of the LCG in closed form: s_k = A^k s_0 + C (A^k-1)/(A-1) mod 2^64."""
    ak = pow(_A, k, _M * (_A - 1))
    s = (ak * seed + _C * ((ak - 1) // (_A - 1))) % _M
    return np.float32(s >> 40) / np.float32(1 << 24)


def test_weights_init_draw_order_and_values():
    dm, ds, dc, ex, L, idim, seed = 32, 8, 4, 2, 2, 5, 42
    P = orc.M1Params(dm, ds, dc, ex, L, idim, seed=seed)
    di, dr, xd = P.di, P.dr, P.xd

    def kaiming(k, fan_in):
        bound = np.sqrt(np.float32(3.0) / np.float32(fan_in))
        return -bound + np.float32(2.0) * bound * _lcg_draw(seed, k)

    # first draw is input_proj_w[0,0] (src/weights.rs:116), fan_in = input_dim
    assert P.input_proj_w[0, 0] == kaiming(1, idim)
    per_layer = dm * 2 * di + di * dc + di * xd + dr * di + di + di * dm
    k0 = idim * dm
    for l in range(L):
        base = k0 + l * per_layer
        lw = P.layers[l]
        assert lw["in_proj_w"].ravel()[0] == kaiming(base + 1, dm)
        assert lw["conv1d_weight"].ravel()[0] == kaiming(base + dm * 2 * di + 1, dc)
        assert lw["x_proj_w"].ravel()[-1] == kaiming(base + dm * 2 * di + di * dc + di * xd, di)
        kdt = base + dm * 2 * di + di * dc + di * xd
        assert lw["dt_proj_w"].ravel()[0] == kaiming(kdt + 1, dr)
        # dt bias: inv_softplus(exp(U (ln .1 - ln .001) + ln .001)), src/weights.rs:135-140
        uval = float(_lcg_draw(seed, kdt + dr * di + 1))
        dt = math.exp(uval * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
        assert abs(lw["dt_proj_b"][0] - math.log(math.expm1(dt))) < 2e-5 * abs(math.log(math.expm1(dt)))
        assert lw["out_proj_w"].ravel()[0] == kaiming(kdt + dr * di + di + 1, di)
        assert np.all(lw["norm_weight"] == 1) and np.all(lw["d_param"] == 1) and np.all(lw["conv1d_bias"] == 0)
        assert np.allclose(lw["a_neg"], -np.arange(1, ds + 1, dtype=np.float32)[None], rtol=3e-7)
        assert np.allclose(lw["a_log"], np.log(np.arange(1, ds + 1, dtype=np.float64))[None], rtol=2e-7, atol=0)
        dtv = np.log1p(np.exp(lw["dt_proj_b"].astype(np.float64)))
        assert dtv.min() >= 1e-3 * 0.999 and dtv.max() <= 1e-1 * 1.001
        for name, fan in (("in_proj_w", dm), ("conv1d_weight", dc), ("x_proj_w", di), ("dt_proj_w", dr), ("out_proj_w", di)):
            assert np.abs(lw[name]).max() <= math.sqrt(3.0 / fan) * (1 + 1e-6)
    assert np.all(P.norm_f_weight == 1) and np.all(P.input_proj_b == 0)


# ----------------------------------------------------------------- backbone --
def _np_layer_step(x, lw, conv_win, h, P, eps):
    """Independent float64 numpy statement of one layer for one token (the per-layer
    maths of src/mamba_ssm/cpu/inference.rs:88-268, written from the equations).
    conv_win: [di, dc-1] previous inputs oldest first; h: [di, ds]."""
    di, ds, dr, dc = P.di, P.ds, P.dr, P.dc
    w = {k: v.astype(np.float64) for k, v in lw.items()}
    n = x / np.sqrt(np.mean(x * x) + eps) * w["norm_weight"]
    proj = n @ w["in_proj_w"]
    xb, z = proj[:di], proj[di:]
    g = z / (1 + np.exp(-z))
    win = np.concatenate([conv_win, xb[:, None]], axis=1)            # [di, dc]
    c = (win * w["conv1d_weight"]).sum(1) + w["conv1d_bias"]
    u = c / (1 + np.exp(-c))
    xdbl = u @ w["x_proj_w"]
    dt_raw, Bv, Cv = xdbl[:dr], xdbl[dr:dr + ds], xdbl[dr + ds:]
    draw = dt_raw @ w["dt_proj_w"] + w["dt_proj_b"]
    delta = np.where(draw > 20, draw, np.log1p(np.exp(draw)))
    h_new = np.exp(delta[:, None] * w["a_neg"]) * h + (delta * u)[:, None] * Bv[None]
    y = h_new @ Cv + w["d_param"] * u
    out = (y * g) @ w["out_proj_w"]
    return x + out, win[:, 1:], h_new


def test_backbone_step_matches_independent_numpy():
    dm, ds, dc, ex, L, idim = 32, 8, 4, 2, 2, 6
    P = orc.M1Params(dm, ds, dc, ex, L, idim, seed=7)
    rng = np.random.default_rng(30)
    conv, ssm = orc.m1_zero_state(P)
    wins = [np.zeros((P.di, dc - 1)) for _ in range(L)]
    hs = [np.zeros((P.di, ds)) for _ in range(L)]
    for t in range(6):
        x = rng.standard_normal(idim).astype(np.float32)
        got = orc.m1_backbone_step(P, x, conv, ssm)
        r = x.astype(np.float64) @ P.input_proj_w.astype(np.float64) + P.input_proj_b
        for l in range(L):
            r, wins[l], hs[l] = _np_layer_step(r, P.layers[l], wins[l], hs[l], P, 1e-5)
        want = r / np.sqrt(np.mean(r * r) + 1e-5) * P.norm_f_weight
        assert scaled_err(got, want) < 2e-5, t
        for l in range(L):
            assert scaled_err(ssm[l].reshape(P.di, ds), hs[l]) < 2e-5
            assert np.allclose(conv[l].reshape(P.di, dc - 1), wins[l], atol=1e-5)


def _cfg_small():
    # tests/prefill.rs:37-47 test_cfg: d_model 32, 2 layers, d_state 8, d_conv 4, expand 2
    return dict(dm=32, ds=8, dc=4, expand=2, n_layers=2)


def test_prefill_then_step_equals_step_loop():
    # tests/prefill.rs:173-232: prefill T then one step == T+1 steps (cos > 0.9999, max_rel < 1e-2)
    c = _cfg_small(); idim = 12; T = 24
    P = orc.M1Params(c["dm"], c["ds"], c["dc"], c["expand"], c["n_layers"], idim, seed=1234)
    x = det((T + 1) * idim, 11, 2.0).reshape(T + 1, idim)
    conv_a, ssm_a = orc.m1_zero_state(P)
    for t in range(T + 1):
        out_a = orc.m1_backbone_step(P, x[t], conv_a, ssm_a)
    conv_b, ssm_b = orc.m1_zero_state(P)
    pre = orc.m1_backbone_prefill(P, x[:T], conv_b, ssm_b, threads=1)
    out_b = orc.m1_backbone_step(P, x[T], conv_b, ssm_b)
    assert cosine(out_a, out_b) > 0.9999 and max_rel(out_b, out_a, floor=1e-3) < 1e-2
    assert scaled_err(ssm_b, ssm_a) < 1e-4 and np.allclose(conv_b, conv_a, atol=1e-5)
    # every prefill position equals the step loop's output at that position
    conv_c, ssm_c = orc.m1_zero_state(P)
    for t in range(T):
        o = orc.m1_backbone_step(P, x[t], conv_c, ssm_c)
        assert cosine(o, pre[t]) > 0.9999


def test_prefill_parallel_equals_single_bitwise_and_chunked_carry():
    # tests/prefill.rs:136-168 (Parallel == Single incl. conv/ssm state)
    c = _cfg_small(); idim = 32; T = 40
    P = orc.M1Params(c["dm"], c["ds"], c["dc"], c["expand"], c["n_layers"], idim, seed=99)
    x = det(T * idim, 5, 2.0).reshape(T, idim)
    c1, s1 = orc.m1_zero_state(P); o1 = orc.m1_backbone_prefill(P, x, c1, s1, threads=1)
    c8, s8 = orc.m1_zero_state(P); o8 = orc.m1_backbone_prefill(P, x, c8, s8, threads=8)
    assert np.array_equal(o1, o8) and np.array_equal(c1, c8) and np.array_equal(s1, s8)
    # two prefills with carried state == one prefill (state handoff is exact in this route)
    ca, sa = orc.m1_zero_state(P)
    oa = orc.m1_backbone_prefill(P, x[:17], ca, sa, threads=1)
    ob = orc.m1_backbone_prefill(P, x[17:], ca, sa, threads=1)
    assert np.array_equal(np.concatenate([oa, ob]), o1) and np.array_equal(sa, s1) and np.array_equal(ca, c1)


def test_identity_input_proj_equals_eye_projection():
    # tests/prefill.rs:236-311: empty input_proj (identity copy) == explicit eye GEMM, bitwise
    c = _cfg_small(); dm = c["dm"]; T = 10
    P = orc.M1Params(dm, c["ds"], c["dc"], c["expand"], c["n_layers"], dm, seed=3)
    P.input_proj_w[:] = np.eye(dm, dtype=np.float32)
    P.input_proj_b[:] = 0
    x = det(T * dm, 21, 2.0).reshape(T, dm)
    ca, sa = orc.m1_zero_state(P); oa = orc.m1_backbone_prefill(P, x, ca, sa, identity_proj=True, threads=1)
    cb, sb = orc.m1_zero_state(P); ob = orc.m1_backbone_prefill(P, x, cb, sb, identity_proj=False, threads=1)
    assert np.array_equal(oa, ob) and np.array_equal(sa, sb)


def test_step_state_carries_and_reset_reproduces():
    # tests/m1_test_correctness.rs:17-146
    P = orc.M1Params(128, 16, 4, 2, 2, 128, seed=42)   # the tiny CPU configuration
    x = det(128, 3, 2.0)
    conv, ssm = orc.m1_zero_state(P)
    o1 = orc.m1_backbone_step(P, x, conv, ssm)
    o2 = orc.m1_backbone_step(P, x, conv, ssm)
    assert np.any(o1 != 0) and np.max(np.abs(o1 - o2)) > 1e-6        # state carries
    conv[:] = 0; ssm[:] = 0
    o3 = orc.m1_backbone_step(P, x, conv, ssm)
    assert np.array_equal(o1, o3)                                     # reset reproduces
