"""GPU parity at seeded random shapes: the selective scan on each of its routes, conv1d + SiLU over a sequence, and both
engines' prefill followed by hand-off steps, against the f64 oracle / the CPU route.  The fixed-shape tests pick their
shapes for a reason each; these draw them (odd lengths around the kernels' tile sizes, channel counts off the 64-channel
tile, every storage type and route) so that a shape nobody thought of has a chance of being in the suite."""
import numpy as np
import pytest
import torch

import orc
from gpu_util import DEV, assert_close, dev, host, quant
from util import cosine, scaled_err, scan_inputs

pytestmark = pytest.mark.gpu

ops = pytest.importorskip("mamba_rs_amd.ops")
from mamba_rs_amd import (GpuMamba3Backbone, GpuMambaBackbone, Mamba3Config, MambaConfig, MambaWeights,  # noqa: E402
                          WeightDtype)
import test_engine_gpu as m1e  # noqa: E402
import test_m3_engine_gpu as m3e  # noqa: E402
from test_m1_scan_gpu import run_scan  # noqa: E402

ROUND = {WeightDtype.F32: None, WeightDtype.BF16: orc.BF16, WeightDtype.F16: orc.F16}


@pytest.mark.parametrize("seed", range(16))
def test_scan_at_a_random_shape(seed):
    rng = np.random.default_rng(1000 + seed)
    batch = int(rng.integers(1, 6))
    T = int(rng.choice([2, 3, 5, 17, 63, 64, 65, 127, 129, 255, 257, 300, 511, 640, 777, 1025]))
    di = int(rng.choice([8, 24, 40, 64, 72, 128, 136, 200, 256, 320]))
    dtype = int(rng.choice([orc.F32, orc.BF16, orc.F16]))
    s4d, gate = bool(rng.integers(0, 2)), int(rng.integers(0, 3))
    route = str(rng.choice(["force", "auto", "none"]))
    ds = 16 if route != "none" else int(rng.choice([4, 8, 16, 24, 64]))
    if route == "force" and T < 64:
        route = "auto"
    print(f"case scan B={batch} T={T} di={di} ds={ds} dtype={dtype} s4d={s4d} gate={gate} route={route}", flush=True)
    inp = scan_inputs(rng, batch, T, di, ds, s4d=s4d)
    for k in ("u", "delta", "B", "C", "z"):
        inp[k] = quant(inp[k], dtype)
    h0 = (rng.standard_normal((batch, di, ds)) * 0.1).astype(np.float32)
    y_ref, h_ref = orc.m1_scan_f64(h0, inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"],
                                   gate=inp["z"] if gate else None, gate_mode=gate)
    y, h = run_scan(inp, h0, dtype, gate, flags=ops.A_S4D_REAL if s4d else 0, split=None if route == "none" else route)
    assert_close(y, y_ref, dtype, "y")
    assert_close(h, h_ref, orc.F32, "h")


@pytest.mark.parametrize("seed", range(16))
def test_conv_over_a_sequence_at_a_random_shape(seed):
    rng = np.random.default_rng(2000 + seed)
    batch = int(rng.integers(1, 5))
    T = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 33, 100, 257, 600]))
    di = int(rng.choice([4, 8, 20, 64, 100, 200, 256, 260, 516]))
    dc = int(rng.choice([2, 3, 4, 4, 4]))
    dtype = int(rng.choice([orc.F32, orc.BF16, orc.F16]))
    wide = bool(rng.integers(0, 2))   # x read in place out of rows twice as wide (the x half of in_proj's output)
    print(f"case conv B={batch} T={T} di={di} dc={dc} dtype={dtype} wide={wide}", flush=True)
    full = quant(rng.standard_normal((batch, T, 2 * di if wide else di)).astype(np.float32), dtype)
    w = (rng.standard_normal((di, dc)) * 0.5).astype(np.float32)
    bias = (rng.standard_normal(di) * 0.1).astype(np.float32)
    st0 = rng.standard_normal((batch, di, dc)).astype(np.float32)
    out_ref, st_ref = orc.conv1d_seq_f64(st0, np.ascontiguousarray(full[:, :, :di]), w, bias)
    st, fd = dev(st0), dev(full, dtype)
    u = torch.empty(batch, T, di, device=DEV, dtype=fd.dtype)
    ops.conv1d_seq_silu(u, st, fd[:, :, :di], dev(w), dev(bias))
    assert_close(host(u), out_ref, dtype, "u")
    assert np.array_equal(host(st), st_ref.astype(np.float32)), "window state"


def _held(got, want, dtype, what, f32_bar):
    if dtype == WeightDtype.F32:
        assert scaled_err(got, want) < f32_bar, (what, scaled_err(got, want))
    else:
        assert cosine(got, want) >= 0.999, (what, cosine(got, want))


@pytest.mark.parametrize("seed", range(10))
def test_mamba1_engine_prefill_and_steps_at_a_random_shape(seed):
    rng = np.random.default_rng(3000 + seed)
    dm = int(rng.choice([64, 128, 192, 256]))
    cfg = MambaConfig(d_model=dm, d_state=int(rng.choice([8, 16, 16, 16, 32])), d_conv=int(rng.choice([2, 3, 4, 4])),
                      expand=int(rng.choice([1, 2, 2])), n_layers=int(rng.integers(1, 4)))
    B, T = int(rng.integers(1, 5)), int(rng.choice([2, 3, 7, 31, 32, 33, 64, 100, 257, 300, 513]))
    dtype = [WeightDtype.F32, WeightDtype.BF16, WeightDtype.F16][int(rng.integers(0, 3))]
    idim = int(rng.choice([dm, 24, 40]))
    print(f"case m1 engine {cfg} B={B} T={T} dtype={dtype} input_dim={idim}", flush=True)
    w = MambaWeights.init(cfg, idim, 100 + seed)
    P = m1e.oracle_params(w, cfg, idim, round_to=ROUND[dtype])
    xs = (rng.standard_normal((B, T + 3, idim)) * 0.5).astype(np.float32)
    eng = GpuMambaBackbone.new_with_dtype(0, w, cfg, idim, B, dtype)
    last = eng.prefill_sequence(xs[:, :T])
    outs = [eng.step(xs[:, T + k]).copy() for k in range(3)]
    eng.close()
    b = int(rng.integers(0, B))
    conv, ssm = orc.m1_zero_state(P)
    _held(last[b], orc.m1_backbone_prefill(P, xs[b, :T], conv, ssm)[-1], dtype, "prefill", 2e-4)
    for k in range(3):
        _held(outs[k][b], orc.m1_backbone_step(P, xs[b, T + k], conv, ssm), dtype, f"step {k}", 2e-4)


@pytest.mark.parametrize("seed", range(10))
def test_mamba3_engine_prefill_and_steps_at_a_random_shape(seed):
    rng = np.random.default_rng(4000 + seed)
    hd, ds = [(16, 16), (16, 64), (32, 32), (64, 64), (32, 64), (64, 16)][int(rng.integers(0, 6))]   # headdim x d_state / 4: whole waves
    dm = int(rng.choice([64, 128, 192]))
    nh = 2 * dm // hd
    ng = int(rng.choice([g for g in (1, 2, 3, 4) if nh % g == 0]))
    cfg = Mamba3Config(d_model=dm, d_state=ds, expand=2, headdim=hd, ngroups=ng, n_layers=int(rng.integers(1, 4)),
                       rope_fraction=float(rng.choice([0.5, 1.0])), is_outproj_norm=bool(rng.integers(0, 2)))
    B, T = int(rng.integers(1, 4)), int(rng.choice([2, 5, 63, 64, 65, 130, 257, 400]))
    dtype = [WeightDtype.F32, WeightDtype.BF16][int(rng.integers(0, 2))]
    idim = int(rng.choice([dm, 24]))
    print(f"case m3 engine {cfg} B={B} T={T} dtype={dtype} input_dim={idim}", flush=True)
    w = m3e.perturbed(cfg, idim, 200 + seed)
    P = m3e.oracle_params(w, cfg, idim, round_to=ROUND[dtype])
    xs = (rng.standard_normal((B, T + 3, idim)) * 0.5).astype(np.float32)
    eng = GpuMamba3Backbone.new_with_dtype(0, w, cfg, idim, B, dtype)
    last = eng.prefill_sequence(xs[:, :T])
    outs = [eng.step(xs[:, T + k]).copy() for k in range(3)]
    eng.close()
    b = int(rng.integers(0, B))
    st = P.zero_state()
    ref = None
    for t in range(T):
        ref = orc.m3_backbone_step(P, xs[b, t], st)
    _held(last[b], ref, dtype, "prefill", 5e-4)
    for k in range(3):
        _held(outs[k][b], orc.m3_backbone_step(P, xs[b, T + k], st), dtype, f"step {k}", 5e-4)
