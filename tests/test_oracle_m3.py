"""Pins for the Mamba-3 SISO part of the CPU oracle (oracle/m3_oracle.c). CPU only.

The reference holds no golden vectors; the sequential recurrence is pinned by closed forms
and an independent numpy brute force, the chunked algebra by the chunked == sequential
identity (the relation tests/m3_cpu_gpu_train_parity.rs:60-66 checks across routes), and the
per-layer step by an independent float64 numpy statement of the equations plus the
reference's unit-test invariants (src/mamba3_siso/cpu/inference.rs:367-617).
"""
import math

import numpy as np
import pytest

import orc
from util import cosine, scaled_err


def m3_inputs(rng, B, T, nh, hd, ds):
    """Scan-level inputs with realistic ranges: dt = softplus(...) in ~[1e-3, 0.3], a_val <= -a_floor,
    trap in (0,1), K/Q ~ N(0,1)+1 (bias 1, as initialised), x ~ N(0,1)."""
    x = rng.standard_normal((B, T, nh * hd)).astype(np.float32)
    K = (rng.standard_normal((B, T, nh, ds)) + 1.0).astype(np.float32)
    Q = (rng.standard_normal((B, T, nh, ds)) + 1.0).astype(np.float32)
    dt = np.log1p(np.exp(rng.standard_normal((B, T, nh)) - 3.0)).astype(np.float32)
    v = rng.standard_normal((B, T, nh)).astype(np.float32)
    a_val = np.minimum(-np.where(v >= 0, 1 + v, 1 / (1 - v)), -1e-4).astype(np.float32)
    trap = (1 / (1 + np.exp(-rng.standard_normal((B, T, nh))))).astype(np.float32)
    D = rng.uniform(0.5, 1.5, nh).astype(np.float32)
    return dict(x=x, K=K, Q=Q, dt=dt, a_val=a_val, trap=trap, D=D)


def zero_state(B, nh, hd, ds):
    return np.zeros((B, nh, hd, ds)), np.zeros((B, nh, ds)), np.zeros((B, nh, hd))


def _np_seq(ssm, kst, vst, inp):
    """Independent numpy statement of the trapezoid (einsum per step), float64."""
    x, K, Q = (inp[k].astype(np.float64) for k in ("x", "K", "Q"))
    B, T, nh, ds = K.shape
    hd = x.shape[2] // nh
    al = np.exp(inp["a_val"].astype(np.float64) * inp["dt"].astype(np.float64))
    be = al * inp["dt"] * (1.0 - inp["trap"].astype(np.float64))
    ga = inp["trap"].astype(np.float64) * inp["dt"]
    H, kp, vp = ssm.copy(), kst.copy(), vst.copy()
    y = np.zeros_like(x)
    for t in range(T):
        xt = x[:, t].reshape(B, nh, hd)
        H = al[:, t, :, None, None] * H + be[:, t, :, None, None] * vp[..., None] * kp[:, :, None, :] \
            + ga[:, t, :, None, None] * xt[..., None] * K[:, t][:, :, None, :]
        y[:, t] = (np.einsum("bhpn,bhn->bhp", H, Q[:, t]) + inp["D"][None, :, None] * xt).reshape(B, nh * hd)
        kp, vp = K[:, t].copy(), xt.copy()
    return y, H, kp, vp


def test_abg_formulas():
    rng = np.random.default_rng(1)
    inp = m3_inputs(rng, 2, 5, 3, 4, 4)
    al, be, ga = orc.m3_abg_f64(inp["dt"], inp["a_val"], inp["trap"])
    assert np.allclose(al, np.exp(inp["a_val"].astype(np.float64) * inp["dt"]), rtol=1e-14)
    assert np.allclose(be, al * inp["dt"] * (1 - inp["trap"].astype(np.float64)), rtol=1e-14)
    assert np.allclose(ga, inp["trap"].astype(np.float64) * inp["dt"], rtol=1e-14)


def test_seq_f64_matches_independent_numpy():
    rng = np.random.default_rng(2)
    B, T, nh, hd, ds = 2, 11, 3, 4, 6
    inp = m3_inputs(rng, B, T, nh, hd, ds)
    ssm0 = rng.standard_normal((B, nh, hd, ds)) * 0.2
    k0 = rng.standard_normal((B, nh, ds)); v0 = rng.standard_normal((B, nh, hd))
    al, be, ga = orc.m3_abg_f64(inp["dt"], inp["a_val"], inp["trap"])
    y, ssm, kst, vst = orc.m3_seq_f64(ssm0, k0, v0, inp["x"], inp["K"], inp["Q"], al, be, ga, inp["D"])
    yn, Hn, kn, vn = _np_seq(ssm0, k0, v0, inp)
    assert np.allclose(y, yn, atol=1e-12) and np.allclose(ssm, Hn, atol=1e-12)
    assert np.array_equal(kst, kn) and np.array_equal(vst, vn)


def test_seq_special_cases():
    rng = np.random.default_rng(3)
    B, T, nh, hd, ds = 1, 6, 2, 3, 4
    inp = m3_inputs(rng, B, T, nh, hd, ds)
    z = zero_state(B, nh, hd, ds)
    ones = np.ones((B, T, nh)); zeros = np.zeros((B, T, nh))
    # alpha = 1, beta = 0, gamma = 1: H is the running sum of x k^T
    y, ssm, _, _ = orc.m3_seq_f64(*z, inp["x"], inp["K"], inp["Q"], ones, zeros, ones, inp["D"])
    want = np.einsum("btp,btn->pn", inp["x"][:, :, :hd].astype(np.float64), inp["K"][:, :, 0].astype(np.float64))
    assert np.allclose(ssm[0, 0], want, atol=1e-12)
    # trap = 1 (beta = 0, gamma = dt): a Mamba-2 style update h = alpha h + dt x k^T; k/v history is irrelevant
    inp1 = dict(inp); inp1["trap"] = np.ones_like(inp["trap"])
    al, be, ga = orc.m3_abg_f64(inp1["dt"], inp1["a_val"], inp1["trap"])
    assert np.all(be == 0) and np.allclose(ga, inp1["dt"])
    ya, sa, _, _ = orc.m3_seq_f64(*z, inp["x"], inp["K"], inp["Q"], al, be, ga, inp["D"])
    k0 = rng.standard_normal((B, nh, ds)); v0 = rng.standard_normal((B, nh, hd))
    yb, sb, _, _ = orc.m3_seq_f64(z[0], k0, v0, inp["x"], inp["K"], inp["Q"], al, be, ga, inp["D"])
    assert np.array_equal(ya, yb) and np.array_equal(sa, sb)
    # two calls with carried state == one call (state handoff is exact)
    al, be, ga = orc.m3_abg_f64(inp["dt"], inp["a_val"], inp["trap"])
    y, s, k, v = orc.m3_seq_f64(*z, inp["x"], inp["K"], inp["Q"], al, be, ga, inp["D"])
    y1, s1, k1, v1 = orc.m3_seq_f64(*z, inp["x"][:, :4], inp["K"][:, :4], inp["Q"][:, :4], al[:, :4], be[:, :4], ga[:, :4], inp["D"])
    y2, s2, k2, v2 = orc.m3_seq_f64(s1, k1, v1, inp["x"][:, 4:], inp["K"][:, 4:], inp["Q"][:, 4:], al[:, 4:], be[:, 4:], ga[:, 4:], inp["D"])
    assert np.array_equal(np.concatenate([y1, y2], 1), y) and np.array_equal(s2, s)


def test_seq_gpu_route_tracks_f64():
    rng = np.random.default_rng(4)
    B, T, nh, hd, ds = 2, 64, 4, 8, 16
    inp = m3_inputs(rng, B, T, nh, hd, ds)
    al, be, ga = orc.m3_abg_f64(inp["dt"], inp["a_val"], inp["trap"])
    z = zero_state(B, nh, hd, ds)
    y, s, _, _ = orc.m3_seq_f64(*z, inp["x"], inp["K"], inp["Q"], al, be, ga, inp["D"])
    yg, sg, _, _ = orc.m3_seq_gpu(*z, inp["x"], inp["K"], inp["Q"], al, be, ga, inp["D"])
    assert scaled_err(yg, y) < 3e-6 and scaled_err(sg, s) < 3e-6


@pytest.mark.parametrize("T,cs", [(10, 4), (64, 64), (130, 64), (7, 16), (33, 8)])
@pytest.mark.parametrize("carry", [False, True])
def test_chunked_equals_sequential(T, cs, carry):
    """tests/m3_chunked_fwd_unit_parity.rs uses B=2, T=10, chunk 4 (partial last chunk)."""
    rng = np.random.default_rng(100 + T + cs)
    B, nh, hd, ds = 2, 3, 8, 8
    inp = m3_inputs(rng, B, T, nh, hd, ds)
    if carry:
        st = (rng.standard_normal((B, nh, hd, ds)) * 0.3, rng.standard_normal((B, nh, ds)), rng.standard_normal((B, nh, hd)))
    else:
        st = zero_state(B, nh, hd, ds)
    al, be, ga = orc.m3_abg_f64(inp["dt"], inp["a_val"], inp["trap"])
    y, s, k, v = orc.m3_seq_f64(*st, inp["x"], inp["K"], inp["Q"], al, be, ga, inp["D"])
    yc, sc, kc, vc = orc.m3_chunked_f64(*st, inp["x"], inp["K"], inp["Q"], inp["dt"], inp["trap"], inp["a_val"], inp["D"], cs,
                                        carry=carry)
    assert np.allclose(yc, y, rtol=1e-10, atol=1e-10) and np.allclose(sc, s, rtol=1e-10, atol=1e-10)
    assert np.array_equal(kc, k) and np.array_equal(vc, v)


def test_chunked_stateless_window_ignores_entering_state():
    # kernels/mamba3_chunked.cu:219-223: chunk 0 always enters with zero state
    rng = np.random.default_rng(7)
    B, T, nh, hd, ds = 1, 12, 2, 4, 4
    inp = m3_inputs(rng, B, T, nh, hd, ds)
    st = (rng.standard_normal((B, nh, hd, ds)), rng.standard_normal((B, nh, ds)), rng.standard_normal((B, nh, hd)))
    a = orc.m3_chunked_f64(*st, inp["x"], inp["K"], inp["Q"], inp["dt"], inp["trap"], inp["a_val"], inp["D"], 4, carry=False)
    b = orc.m3_chunked_f64(*zero_state(B, nh, hd, ds), inp["x"], inp["K"], inp["Q"], inp["dt"], inp["trap"], inp["a_val"], inp["D"], 4)
    assert all(np.array_equal(u, v) for u, v in zip(a, b))


# ------------------------------------------------------------------ weights --
def _xorshift_draws(seed, n):
    s = max(seed, 1); out = []
    for _ in range(n):
        s ^= (s << 13) & 0xFFFFFFFFFFFFFFFF; s ^= s >> 7; s ^= (s << 17) & 0xFFFFFFFFFFFFFFFF
        out.append(np.float32(s & 0xFFFFFF) / np.float32(16777216.0))
    return out


def test_m3_weights_init_order_and_constants():
    P = orc.M3Params(16, 8, 2, 8, 1, 2, 0.5, 3, seed=11)
    dm, di, nh, ip, idim = 16, 32, 4, P.ip, 3
    assert ip == 2 * di + 2 * 8 + 3 * nh + 2 and P.n_rope == 2            # config.rs:30-58
    n_first = idim * dm + dm * ip + di * dm + nh
    dr = _xorshift_draws(11, n_first + 1)
    b = np.float32(math.sqrt(3.0 / idim))
    assert P.input_proj_w.ravel()[0] == (dr[0] * np.float32(2) - np.float32(1)) * b
    l0 = P.layers[0]
    assert l0["in_proj_w"].ravel()[0] == (dr[idim * dm] * np.float32(2) - np.float32(1)) * np.float32(math.sqrt(3.0 / dm))
    assert l0["out_proj_w"].ravel()[0] == (dr[idim * dm + dm * ip] * np.float32(2) - np.float32(1)) * np.float32(math.sqrt(3.0 / di))
    uval = float(dr[idim * dm + dm * ip + di * dm])                       # dt_bias after out_proj (weights.rs:130-139)
    dtv = math.exp(uval * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
    assert abs(l0["dt_bias"][0] - math.log(math.expm1(dtv))) < 2e-5 * abs(math.log(math.expm1(dtv)))
    # next layer continues the same stream
    assert P.layers[1]["in_proj_w"].ravel()[0] == (dr[n_first] * np.float32(2) - np.float32(1)) * np.float32(math.sqrt(3.0 / dm))
    for lw in P.layers:
        for name in ("norm_weight", "b_norm_weight", "c_norm_weight", "b_bias", "c_bias", "d_param", "norm_gate_weight"):
            assert np.all(lw[name] == 1.0), name
    assert np.all(P.norm_f_weight == 1) and np.all(P.input_proj_b == 0)


# --------------------------------------------------------------- layer step --
def _np_m3_layer(r, lw, st, P):
    """Independent float64 numpy statement of one Mamba-3 layer for one token."""
    H, kp, vp, ang = st
    di, nh, hd, ds, ng, nr = P.di, P.nh, P.hd, P.ds, P.ng, P.n_rope
    w = {k: v.astype(np.float64) for k, v in lw.items()}
    eps = 1e-5
    n = r / np.sqrt(np.mean(r * r) + eps) * w["norm_weight"]
    proj = n @ w["in_proj_w"]
    o = 0
    z = proj[o:o + di]; o += di
    x = proj[o:o + di]; o += di
    Braw = proj[o:o + ng * ds].reshape(ng, ds); o += ng * ds
    Craw = proj[o:o + ng * ds].reshape(ng, ds); o += ng * ds
    dd_dt = proj[o:o + nh]; o += nh
    dd_a = proj[o:o + nh]; o += nh
    trp = proj[o:o + nh]; o += nh
    theta = proj[o:o + nr]
    Bn = Braw / np.sqrt((Braw ** 2).mean(1, keepdims=True) + eps) * w["b_norm_weight"]
    Cn = Craw / np.sqrt((Craw ** 2).mean(1, keepdims=True) + eps) * w["c_norm_weight"]
    y = np.zeros(di)
    Hn, kn, vn, an = H.copy(), kp.copy(), vp.copy(), ang.copy()
    for h in range(nh):
        g = h // (nh // ng)
        ht = 1 + dd_a[h] if dd_a[h] >= 0 else 1 / (1 - dd_a[h])
        A = min(-ht, -P.a_floor)
        v = dd_dt[h] + w["dt_bias"][h]
        dt = v if v > 20 else np.log1p(np.exp(v))
        k = Bn[g] + w["b_bias"][h]; q = Cn[g] + w["c_bias"][h]
        for a in range(nr):
            phi = (ang[h, a] + np.tanh(theta[a]) * np.pi * dt) % (2 * np.pi)
            an[h, a] = phi
            c, s = np.cos(phi), np.sin(phi)
            k[2 * a], k[2 * a + 1] = c * k[2 * a] - s * k[2 * a + 1], s * k[2 * a] + c * k[2 * a + 1]
            q[2 * a], q[2 * a + 1] = c * q[2 * a] - s * q[2 * a + 1], s * q[2 * a] + c * q[2 * a + 1]
        al = np.exp(A * dt); tau = 1 / (1 + np.exp(-trp[h])); be = al * dt * (1 - tau); ga = tau * dt
        xh = x[h * hd:(h + 1) * hd]
        Hn[h] = al * H[h] + be * np.outer(vp[h], kp[h]) + ga * np.outer(xh, k)
        y[h * hd:(h + 1) * hd] = Hn[h] @ q + w["d_param"][h] * xh
        kn[h], vn[h] = k, xh
    if P.outproj_norm:
        yg = y.reshape(nh, hd)
        gated = (yg / np.sqrt((yg ** 2).mean(1, keepdims=True) + eps)).reshape(di) * w["norm_gate_weight"] * z / (1 + np.exp(-z))
    else:
        gated = y * z / (1 + np.exp(-z))
    return r + gated @ w["out_proj_w"], (Hn, kn, vn, an)


@pytest.mark.parametrize("outproj_norm", [False, True])
def test_m3_backbone_step_matches_independent_numpy(outproj_norm):
    P = orc.M3Params(32, 16, 2, 16, 2, 2, 0.5, 6, seed=21, outproj_norm=outproj_norm)
    rng = np.random.default_rng(5)
    st = P.zero_state()
    nst = [(np.zeros((P.nh, P.hd, P.ds)), np.zeros((P.nh, P.ds)), np.zeros((P.nh, P.hd)), np.zeros((P.nh, P.n_rope)))
           for _ in range(P.n_layers)]
    for t in range(5):
        x = rng.standard_normal(6).astype(np.float32)
        got, taps = orc.m3_backbone_step(P, x, st, taps=True)
        r = x.astype(np.float64) @ P.input_proj_w.astype(np.float64) + P.input_proj_b
        for l in range(P.n_layers):
            r, nst[l] = _np_m3_layer(r, P.layers[l], nst[l], P)
        want = r / np.sqrt(np.mean(r * r) + 1e-5) * P.norm_f_weight
        assert scaled_err(got, want) < 3e-5, t
        for l in range(P.n_layers):
            assert scaled_err(st[0][l], nst[l][0]) < 3e-5 and scaled_err(st[1][l], nst[l][1]) < 3e-5
            ang = st[3][l][:, :P.n_rope]
            assert np.all(ang >= 0) and np.all(ang < 2 * np.pi + 1e-6)          # cpu/inference.rs tests: angle in [0, 2pi)
            d = np.abs(ang - nst[l][3]); d = np.minimum(d, 2 * np.pi - d)
            assert d.max() < 1e-4
            # taps are consistent with the abg formulas
            al, be, ga = orc.m3_abg_f64(taps[l]["dt"], taps[l]["a_val"], taps[l]["trap"])
            assert np.allclose(taps[l]["alpha"], al, rtol=3e-6) and np.allclose(taps[l]["beta"], be, rtol=3e-6, atol=1e-9)
            assert np.all(taps[l]["a_val"] <= -P.a_floor)


def test_m3_step_determinism_reset_and_rotation_norm():
    # src/mamba3_siso/cpu/inference.rs:367-617: determinism, reset reproduces, state carries
    P = orc.M3Params(128, 16, 2, 16, 1, 4, 0.5, 128, seed=42)       # the reference default config
    x = np.linspace(-1, 1, 128, dtype=np.float32)
    st = P.zero_state()
    o1 = orc.m3_backbone_step(P, x, st)
    o2 = orc.m3_backbone_step(P, x, st)
    assert np.any(o1 != 0) and np.max(np.abs(o1 - o2)) > 1e-7
    st2 = P.zero_state()
    o3 = orc.m3_backbone_step(P, x, st2)
    assert np.array_equal(o1, o3)
    # RoPE is a rotation: |k| per (pair) is preserved -> k_state norm equals the un-rotated k norm (n_rope pairs)
    P0 = orc.M3Params(128, 16, 2, 16, 1, 1, 0.5, 128, seed=42)
    s0 = P0.zero_state()
    _, taps = orc.m3_backbone_step(P0, x, s0, taps=True)
    k = taps[0]["k"]
    lw = P0.layers[0]
    # recompute un-rotated k from the equations
    r = x.astype(np.float64) @ P0.input_proj_w.astype(np.float64)
    n = r / np.sqrt(np.mean(r * r) + 1e-5)
    proj = n @ lw["in_proj_w"].astype(np.float64)
    Braw = proj[2 * P0.di:2 * P0.di + P0.ds]
    k_unrot = Braw / np.sqrt(np.mean(Braw ** 2) + 1e-5) + 1.0
    assert np.allclose(np.linalg.norm(k, axis=1), np.linalg.norm(k_unrot), rtol=1e-5)
    assert np.allclose(k[:, 2 * P0.n_rope:], k_unrot[2 * P0.n_rope:], rtol=1e-5, atol=1e-6)   # indices >= 2*n_rope pass through


def test_python_mamba3_weights_init_equals_the_oracle_restatement():
    """Mamba3Weights.init (numpy, the host mirror) against the oracle's C restatement of weights.rs:120-147: the
    xorshift64 draws and Kaiming scaling bit for bit, dt_bias (exp/log round trip) to 1 ulp."""
    from mamba_rs_amd import Mamba3Config, Mamba3Weights
    cfg = Mamba3Config(d_model=32, d_state=16, expand=2, headdim=16, ngroups=1, n_layers=2, rope_fraction=0.5)
    w = Mamba3Weights.init(cfg, 24, 42)
    P = orc.M3Params(32, 16, 2, 16, 1, 2, 0.5, 24, seed=42)
    assert np.array_equal(w.input_proj_w, P.input_proj_w) and np.array_equal(w.norm_f_weight, P.norm_f_weight)
    for lw, pl in zip(w.layers, P.layers):
        for n in ("norm_weight", "in_proj_w", "b_norm_weight", "c_norm_weight", "b_bias", "c_bias", "d_param", "norm_gate_weight", "out_proj_w"):
            assert np.array_equal(getattr(lw, n), pl[n]), n
        assert np.allclose(lw.dt_bias, pl["dt_bias"], rtol=3e-7, atol=0)
    assert cfg.in_proj_out_dim() == P.ip and cfg.num_rope_angles() == P.n_rope
