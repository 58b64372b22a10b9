"""GPU parity: Mamba-1 selective scan (prefill route) vs the f64 oracle, through the C ABI."""
import numpy as np
import pytest
import torch

import orc
from gpu_util import DEV, assert_close, dev, host, quant
from util import scan_inputs

pytestmark = pytest.mark.gpu

ops = pytest.importorskip("mamba_rs_amd.ops")
from mamba_rs_amd import MambaHipError, _lib  # noqa: E402

GATE_FLAG = {0: ops.GATE_NONE, 1: ops.GATE_PREACT, 2: ops.GATE_SILU}


def run_scan(inp, h0, dtype, gate_mode=0, flags=0, bc_view=None, split=None):
    """Run the HIP scan on quantised inputs; returns (y f32 np, h f32 np).
    split: None = no workspace (sequential route), "auto" = workspace given, "force" = T-split forced."""
    delta, u = dev(inp["delta"], dtype), dev(inp["u"], dtype)
    if bc_view is None:
        Bm, Cm = dev(inp["B"], dtype), dev(inp["C"], dtype)
    else:
        Bm, Cm = bc_view
    a_neg, D = dev(inp["a_neg"]), dev(inp["D"])
    h = dev(h0)
    y = torch.full_like(delta, float("nan"))
    gate = dev(inp["z"], dtype) if gate_mode else None
    workspace = None
    if split is not None:
        batch, T, di = inp["delta"].shape
        workspace = torch.empty(ops.ssm_scan_workspace_bytes(batch, T, di, inp["a_neg"].shape[1]), dtype=torch.uint8, device=DEV)
        if split == "force":
            flags |= ops.FORCE_PARALLEL
    ops.ssm_scan_fwd(h, y, delta, u, Bm, Cm, a_neg, D, gate=gate, flags=flags | GATE_FLAG[gate_mode], workspace=workspace)
    torch.cuda.synchronize()
    return host(y), host(h)


def quantised(rng, batch, T, di, ds, dtype, s4d=True):
    inp = scan_inputs(rng, batch, T, di, ds, s4d=s4d)
    for k in ("u", "delta", "B", "C", "z"):
        inp[k] = quant(inp[k], dtype)
    return inp


SHAPES = [
    # batch, T, d_inner, d_state
    (2, 33, 64, 16),
    (1, 300, 200, 16),    # d_inner not a multiple of the 64-channel tile
    (2, 17, 96, 8),
    (1, 9, 32, 64),       # 4 lanes per channel
    (1, 5, 16, 256),      # reference maximum d_state (src/config.rs:147-152)
    (1, 7, 8, 24),        # d_state not a power of two
    (3, 1, 40, 16),       # T = 1
]


@pytest.mark.parametrize("dtype", [orc.F32, orc.BF16, orc.F16])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("s4d", [False, True])
def test_scan_matches_oracle(shape, dtype, s4d):
    batch, T, di, ds = shape
    rng = np.random.default_rng(hash((shape, dtype, s4d)) & 0xFFFF)
    inp = quantised(rng, batch, T, di, ds, dtype, s4d=s4d)
    h0 = (rng.standard_normal((batch, di, ds)) * 0.1).astype(np.float32)
    for gate_mode in (0, 1, 2):
        print(f"case shape={shape} dtype={dtype} s4d={s4d} gate={gate_mode}", flush=True)
        y_ref, h_ref = orc.m1_scan_f64(h0, inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"],
                                       gate=inp["z"] if gate_mode else None, gate_mode=gate_mode)
        y, h = run_scan(inp, h0, dtype, gate_mode, flags=ops.A_S4D_REAL if s4d else 0)
        assert_close(y, y_ref, dtype, "y")
        assert_close(h, h_ref, orc.F32, "h")


SPLIT_SHAPES = [(2, 333, 64, 16), (1, 300, 200, 16), (3, 64, 128, 16), (1, 1025, 72, 16)]


@pytest.mark.parametrize("dtype", [orc.F32, orc.BF16, orc.F16])
@pytest.mark.parametrize("shape", SPLIT_SHAPES)
@pytest.mark.parametrize("s4d", [False, True])
def test_scan_t_split_route_matches_oracle(shape, dtype, s4d):
    """The chunked (T-split) route: chunk summaries + carry fold must equal the serial scan."""
    batch, T, di, ds = shape
    rng = np.random.default_rng(hash((shape, dtype, s4d, 1)) & 0xFFFF)
    inp = quantised(rng, batch, T, di, ds, dtype, s4d=s4d)
    h0 = (rng.standard_normal((batch, di, ds)) * 0.1).astype(np.float32)
    for gate_mode in (0, 1, 2):
        print(f"case split shape={shape} dtype={dtype} s4d={s4d} gate={gate_mode}", flush=True)
        y_ref, h_ref = orc.m1_scan_f64(h0, inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"],
                                       gate=inp["z"] if gate_mode else None, gate_mode=gate_mode)
        y, h = run_scan(inp, h0, dtype, gate_mode, flags=ops.A_S4D_REAL if s4d else 0, split="force")
        assert_close(y, y_ref, dtype, "y")
        assert_close(h, h_ref, orc.F32, "h")


def test_scan_auto_route_threshold_and_workspace_errors():
    """Up to 256 steps (the reference's serial range, src/config.rs:21-37) the single pass is kept when its (batch row,
    channel tile) pairs fill the machine -- bitwise equal to the no-workspace call -- and MRS_FORCE_SEQUENTIAL keeps it
    in any case; with few pairs the T-split route runs and agrees to the storage tolerance.  A short workspace is refused."""
    rng = np.random.default_rng(9)
    inp = quantised(rng, 16, 64, 4096, 16, orc.BF16)            # 16 x 64 = 1024 pairs
    h0 = np.zeros((16, 4096, 16), np.float32)
    y_seq, h_seq = run_scan(inp, h0, orc.BF16)
    y_auto, h_auto = run_scan(inp, h0, orc.BF16, split="auto")
    assert np.array_equal(y_seq, y_auto) and np.array_equal(h_seq, h_auto)
    inp = quantised(rng, 2, 256, 64, 16, orc.BF16)               # 2 pairs
    h0 = np.zeros((2, 64, 16), np.float32)
    y_seq, h_seq = run_scan(inp, h0, orc.BF16)
    y_forced, h_forced = run_scan(inp, h0, orc.BF16, flags=ops.FORCE_SEQUENTIAL, split="auto")
    assert np.array_equal(y_seq, y_forced) and np.array_equal(h_seq, h_forced)
    y_auto, h_auto = run_scan(inp, h0, orc.BF16, split="auto")
    assert_close(y_auto, y_seq, orc.BF16, "y (auto vs sequential)")
    assert_close(h_auto, h_seq, orc.F32, "h (auto vs sequential)")
    inp = quantised(rng, 2, 512, 64, 16, orc.BF16)
    t = {k: dev(v, orc.BF16 if k in ("u", "delta", "B", "C", "z") else orc.F32) for k, v in inp.items()}
    h = torch.zeros(2, 64, 16, device=DEV); y = torch.empty_like(t["delta"])
    small = torch.empty(256, dtype=torch.uint8, device=DEV)
    with pytest.raises(MambaHipError) as e:
        ops.ssm_scan_fwd(h, y, t["delta"], t["u"], t["B"], t["C"], t["a_neg"], t["D"], workspace=small)
    assert e.value.code == -4


def test_scan_s4d_flag_from_device_check():
    rng = np.random.default_rng(1)
    inp = scan_inputs(rng, 1, 4, 32, 16, s4d=True)
    assert ops.a_neg_is_s4d_real(dev(inp["a_neg"]))
    # a_neg as the reference derives it: -exp(log(n+1)) in f32 (src/weights.rs:44-48,143-148)
    a_log = dev(np.log(np.arange(1, 17, dtype=np.float32))[None].repeat(32, 0))
    a_neg = ops.exp_negate(a_log)
    assert np.allclose(host(a_neg), -np.exp(host(a_log).astype(np.float64)), rtol=3e-7)
    assert ops.a_neg_is_s4d_real(a_neg)
    inp2 = scan_inputs(rng, 1, 4, 32, 16, s4d=False)
    assert not ops.a_neg_is_s4d_real(dev(inp2["a_neg"]))


def test_scan_state_carry_two_calls_equal_one():
    rng = np.random.default_rng(2)
    inp = quantised(rng, 2, 70, 128, 16, orc.BF16)
    h0 = np.zeros((2, 128, 16), np.float32)
    y, h = run_scan(inp, h0, orc.BF16, 2)
    a = {k: (v[:, :41] if v.ndim == 3 and v.shape[1] == 70 else v) for k, v in inp.items()}
    b = {k: (v[:, 41:] if v.ndim == 3 and v.shape[1] == 70 else v) for k, v in inp.items()}
    y1, h1 = run_scan(a, h0, orc.BF16, 2)
    y2, h2 = run_scan(b, h1, orc.BF16, 2)
    assert np.array_equal(np.concatenate([y1, y2], 1), y) and np.array_equal(h2, h)


@pytest.mark.parametrize("dtype", [orc.F32, orc.BF16])
def test_scan_reads_b_c_in_place_from_xdbl(dtype):
    # B and C as strided views of xdbl [batch, T, dt_rank + 2*ds] (130m shape: 48 + 32)
    rng = np.random.default_rng(3)
    batch, T, di, ds, dr = 2, 20, 64, 16, 48
    inp = quantised(rng, batch, T, di, ds, dtype)
    xdbl = quant(rng.standard_normal((batch, T, dr + 2 * ds)).astype(np.float32), dtype)
    inp["B"], inp["C"] = xdbl[:, :, dr:dr + ds].copy(), xdbl[:, :, dr + ds:].copy()
    h0 = np.zeros((batch, di, ds), np.float32)
    xd = dev(xdbl, dtype)
    y, h = run_scan(inp, h0, dtype, 0, bc_view=(xd[:, :, dr:dr + ds], xd[:, :, dr + ds:]))
    y_ref, h_ref = orc.m1_scan_f64(h0, inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"])
    assert_close(y, y_ref, dtype, "y")
    assert_close(h, h_ref, orc.F32, "h")


@pytest.mark.parametrize("shape", [(8, 2048, 1536), (4, 4096, 5120)])
def test_scan_full_size_channel_subset_and_linearity(shape):
    """The isolated-scan workload (B=8, T=2048, d_inner=1536, d_state=16, bf16, gated) and the scan of a 2.8b-shape
    prefill layer (4 x 4096 x 5120: nine chunks of 464 steps over 80 channel tiles): channels are independent, so the
    oracle is run on a subset of channels of the full-size launch, once per A route; plus linearity in u (h0 = 0, f32
    state): scan(2u) = 2 scan(u) exactly."""
    batch, T, di = shape
    ds = 16
    rng = np.random.default_rng(4 + di)
    print(f"case full-size scan {batch} x {T} x {di}", flush=True)
    inp = quantised(rng, batch, T, di, ds, orc.BF16)
    h0 = np.zeros((batch, di, ds), np.float32)
    sel = np.sort(rng.choice(di, 48 if di == 1536 else 24, replace=False))
    sub = dict(delta=inp["delta"][:, :, sel], u=inp["u"][:, :, sel], z=inp["z"][:, :, sel], B=inp["B"], C=inp["C"],
               a_neg=inp["a_neg"][sel], D=inp["D"][sel])
    y_ref, h_ref = orc.m1_scan_f64(h0[:, sel], sub["delta"], sub["u"], sub["B"], sub["C"], sub["a_neg"], sub["D"],
                                   gate=sub["z"], gate_mode=2)
    for flags in (ops.A_S4D_REAL, 0):     # the power-chain kernels and the general-A kernels (a trained checkpoint's)
        y, h = run_scan(inp, h0, orc.BF16, 2, flags=flags, split="auto")
        assert_close(y[:, :, sel], y_ref, orc.BF16, f"y[subset] flags={flags}")
        assert_close(h[:, sel], h_ref, orc.F32, f"h[subset] flags={flags}")
    inp2 = dict(inp); inp2["u"] = inp["u"] * 2.0          # exact in bf16
    y2, h2 = run_scan(inp2, h0, orc.BF16, 0, flags=ops.A_S4D_REAL, split="auto")
    y1, h1 = run_scan(inp, h0, orc.BF16, 0, flags=ops.A_S4D_REAL, split="auto")
    assert np.array_equal(h2, 2.0 * h1) and np.array_equal(y2, 2.0 * y1)


@pytest.mark.parametrize("case", [
    # batch, T, d_inner, dtype, S4D-real, gate mode
    (3, 1000, 320, orc.BF16, True, 2),      # ragged last chunk, partial channel tile
    (2, 300, 192, orc.F32, False, 0),
    (1, 520, 128, orc.F16, True, 1),
    (8, 2048, 1536, orc.BF16, True, 2),     # the benchmark shape
    (4, 4096, 5120, orc.BF16, False, 2),    # the 2.8b-shape layer, general A
])
def test_scan_in_one_launch_equals_the_two_launch_route(case):
    """The T-split route as one launch (every wave summarises its chunk, publishes the summary, waits for the chunks
    before it) against the same two passes as two launches: the arithmetic is the same, so y and the final state must be
    equal bit for bit -- with the flag area cleared by the op itself (the default), and vouched zero by the caller
    (MRS_SCAN_FLAGS_ZERO) on three calls in a row over one workspace, which every call must leave all zero again.
    MRS_FORCE_PARALLEL takes the one launch also where the library would not pick it (general A, few waves)."""
    batch, T, di, dtype, s4d, gate_mode = case
    ds = 16
    rng = np.random.default_rng(T + di)
    print(f"case one-launch scan {case}", flush=True)
    inp = quantised(rng, batch, T, di, ds, dtype, s4d=s4d)
    h0 = (rng.standard_normal((batch, di, ds)) * 0.1).astype(np.float32)
    d = {k: dev(inp[k], dtype) for k in ("u", "delta", "B", "C", "z")}
    a_neg, D = dev(inp["a_neg"]), dev(inp["D"])
    base = GATE_FLAG[gate_mode] | (ops.A_S4D_REAL if s4d else 0)
    gate = d["z"] if gate_mode else None
    ws = torch.empty(ops.ssm_scan_workspace_bytes(batch, T, di, ds), dtype=torch.uint8, device=DEV).fill_(0xA5)
    nflag = ops.ssm_scan_flag_bytes(batch, di)
    assert 0 < nflag < ws.numel()

    def run(extra):
        h, y = dev(h0), torch.full_like(d["delta"], float("nan"))
        ops.ssm_scan_fwd(h, y, d["delta"], d["u"], d["B"], d["C"], a_neg, D, gate=gate, flags=base | extra, workspace=ws)
        torch.cuda.synchronize()
        return y, h

    y2, h2 = run(ops.SCAN_TWO_LAUNCHES)
    assert torch.isfinite(y2.float()).all()
    y1, h1 = run(ops.FORCE_PARALLEL)      # the flags this shape uses are cleared by the op (they held 0xA5 bytes)
    assert torch.equal(y1, y2) and torch.equal(h1, h2)
    ws[:nflag].zero_()                    # what a caller that passes MRS_SCAN_FLAGS_ZERO does once
    for rep in range(3):
        yz, hz = run(ops.SCAN_FLAGS_ZERO | ops.FORCE_PARALLEL)
        assert torch.equal(yz, y2) and torch.equal(hz, h2), rep
        assert int(ws[:nflag].max().item()) == 0, rep


def test_scan_in_one_launch_replays_in_a_graph():
    """The one-launch scan captured in a hipGraph (the static-scratch entry point: no workspace, nothing to clear) and
    replayed with eager calls and synchronisations in between: every replay equals the eager result."""
    rng = np.random.default_rng(77)
    batch, T, di, ds = 2, 700, 256, 16
    inp = quantised(rng, batch, T, di, ds, orc.BF16)
    d = {k: dev(inp[k], orc.BF16) for k in ("u", "delta", "B", "C", "z")}
    a_neg, D = dev(inp["a_neg"]), dev(inp["D"])
    h0 = dev((rng.standard_normal((batch, di, ds)) * 0.1).astype(np.float32))
    flags = ops.GATE_SILU | ops.A_S4D_REAL | ops.FORCE_PARALLEL     # the one launch although the shape is small

    def call(h, y):
        ops.ssm_scan_fwd(h, y, d["delta"], d["u"], d["B"], d["C"], a_neg, D, gate=d["z"], flags=flags, static_scratch=True)

    h_e, y_e = h0.clone(), torch.empty_like(d["delta"])
    call(h_e, y_e)
    torch.cuda.synchronize()
    h_g, y_g = h0.clone(), torch.empty_like(d["delta"])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        call(h_g, y_g)                                  # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(g, stream=side):
            call(h_g, y_g)
    for rep in range(4):
        print(f"case graph replay {rep}", flush=True)
        h_g.copy_(h0); y_g.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_e) and torch.equal(h_g, h_e), rep
        h_x, y_x = h0.clone(), torch.empty_like(d["delta"])
        call(h_x, y_x)                                  # an eager call between replays shares the buffer, in stream order
        torch.cuda.synchronize()
        assert torch.equal(y_x, y_e)


def test_scan_rejects_bad_arguments():
    rng = np.random.default_rng(5)
    inp = quantised(rng, 1, 4, 16, 16, orc.F32)
    t = {k: dev(v) for k, v in inp.items()}
    h = torch.zeros(1, 16, 16, device=DEV)
    y = torch.empty_like(t["delta"])
    s = torch.cuda.current_stream().cuda_stream
    args = [s, 0, h.data_ptr(), y.data_ptr(), t["delta"].data_ptr(), t["u"].data_ptr(), t["B"].data_ptr(),
            t["C"].data_ptr(), t["a_neg"].data_ptr(), t["D"].data_ptr(), 1, 4, 16, 16]

    def expect(code, **chg):
        a = list(args)
        for i, v in chg.items():
            a[int(i[1:])] = v
        with pytest.raises(MambaHipError) as e:
            _lib.call("mrs_ssm_scan_fwd", *a)
        assert e.value.code == code and e.value.message

    expect(-1, _2=None)          # null h
    expect(-3, _1=7)             # dtype
    expect(-2, _13=0)            # d_state 0
    expect(-2, _13=257)          # d_state above the reference maximum
    expect(-2, _11=0)            # T = 0 (src/mamba_ssm/gpu/launch.rs:20-47)
    expect(-2, _10=0)            # batch = 0
    _lib.call("mrs_ssm_scan_fwd", *args)   # and the unmodified call succeeds
    torch.cuda.synchronize()
