"""GPU parity: Mamba-3 SISO step / sequential / chunked-SSD kernels vs the f64 oracle, through the C ABI."""
import numpy as np
import pytest
import torch

import orc
from gpu_util import DEV, REL_TOL, assert_close, dev, host, quant
from test_oracle_m3 import m3_inputs
from util import cosine

pytestmark = pytest.mark.gpu

ops = pytest.importorskip("mamba_rs_amd.ops")


def quantised(rng, B, T, nh, hd, ds, dtype, dt_scale=1.0):
    """dt_scale < 1 slows the decay so that the state carried across chunks (e^{-6} per 64 steps at the
    realistic dt) dominates y instead of vanishing: the cases that pin the inter-chunk algebra."""
    inp = m3_inputs(rng, B, T, nh, hd, ds)
    inp["dt"] = (inp["dt"] * dt_scale).astype(np.float32)
    for k in ("x", "K", "Q"):
        inp[k] = quant(inp[k], dtype)
    return inp


def rand_state(rng, B, nh, hd, ds, dtype, zero=False):
    if zero:
        return (np.zeros((B, nh, hd, ds), np.float32), np.zeros((B, nh, ds), np.float32), np.zeros((B, nh, hd), np.float32))
    # k/v history are earlier activations, so they sit on the storage grid
    return ((rng.standard_normal((B, nh, hd, ds)) * 0.3).astype(np.float32),
            quant(rng.standard_normal((B, nh, ds)).astype(np.float32), dtype),
            quant(rng.standard_normal((B, nh, hd)).astype(np.float32), dtype))


SEQ_SHAPES = [(2, 5, 3, 16, 16), (1, 9, 2, 64, 64), (2, 4, 4, 32, 32), (1, 3, 2, 8, 12), (1, 2, 1, 100, 7), (3, 1, 2, 16, 64)]


@pytest.mark.parametrize("dtype", [orc.F32, orc.BF16, orc.F16])
@pytest.mark.parametrize("shape", SEQ_SHAPES)
def test_m3_seq_and_step_match_oracle(shape, dtype):
    B, T, nh, hd, ds = shape
    rng = np.random.default_rng(hash((shape, dtype)) & 0xFFFF)
    inp = quantised(rng, B, T, nh, hd, ds, dtype)
    st0 = rand_state(rng, B, nh, hd, ds, dtype)
    al64, be64, ga64 = orc.m3_abg_f64(inp["dt"], inp["a_val"], inp["trap"])
    al, be, ga = (v.astype(np.float32) for v in (al64, be64, ga64))
    y_ref, s_ref, k_ref, v_ref = orc.m3_seq_f64(*st0, inp["x"], inp["K"], inp["Q"], al, be, ga, inp["D"])
    print(f"case m3 seq shape={shape} dtype={dtype}", flush=True)
    # device abg vs the formulas
    dal, dbe, dga = ops.m3_compute_abg(dev(inp["dt"]), dev(inp["a_val"]), dev(inp["trap"]))
    assert np.allclose(host(dal), al64, rtol=2e-6) and np.allclose(host(dbe), be64, rtol=2e-6, atol=1e-12) and np.allclose(host(dga), ga64, rtol=1e-6)
    x, K, Q = dev(inp["x"], dtype), dev(inp["K"], dtype), dev(inp["Q"], dtype)
    D = dev(inp["D"])
    # sequence kernel
    ssm, kst, vst = (dev(s) for s in st0)
    y = torch.full_like(x, float("nan"))
    ops.m3_seq_fwd(ssm, kst, vst, y, x, K, Q, dev(al), dev(be), dev(ga), D)
    assert_close(host(y), y_ref, dtype, "y(seq)")
    assert_close(host(ssm), s_ref, orc.F32, "ssm(seq)")
    assert np.array_equal(host(kst), k_ref.astype(np.float32)) and np.array_equal(host(vst), v_ref.astype(np.float32))
    # step kernel, T times
    ssm, kst, vst = (dev(s) for s in st0)
    for t in range(T):
        yt = torch.empty(B, nh * hd, device=DEV, dtype=x.dtype)
        ops.m3_step(ssm, kst, vst, yt, x[:, t].contiguous(), K[:, t].contiguous(), Q[:, t].contiguous(),
                    dev(al[:, t]), dev(be[:, t]), dev(ga[:, t]), D)
        assert_close(host(yt), y_ref[:, t], dtype, f"y(step {t})")
    assert_close(host(ssm), s_ref, orc.F32, "ssm(step)")
    assert np.array_equal(host(kst), k_ref.astype(np.float32)) and np.array_equal(host(vst), v_ref.astype(np.float32))


# the last three are cut into 2, 4 (ragged) and 6 super-chunks when the workspace is passed
SSD_SHAPES = [(2, 10, 3, 16, 16), (2, 130, 3, 16, 16), (1, 256, 2, 64, 64), (1, 200, 2, 32, 64), (1, 64, 1, 64, 16), (2, 65, 2, 16, 32),
              (1, 700, 2, 32, 32), (2, 770, 1, 64, 64)]


def run_ssd(inp, st0, dtype, carry, use_ws=True):
    B, T, nh, ds = inp["K"].shape
    hd = inp["x"].shape[2] // nh
    x, K, Q = dev(inp["x"], dtype), dev(inp["K"], dtype), dev(inp["Q"], dtype)
    ssm, kst, vst = (dev(s) for s in st0)
    y = torch.full_like(x, float("nan"))
    ws = torch.empty(ops.m3_ssd_workspace_bytes(B, T, nh, hd, ds), dtype=torch.uint8, device=DEV) if use_ws else None
    ops.m3_ssd_fwd(ssm, kst, vst, y, x, K, Q, dev(inp["dt"]), dev(inp["trap"]), dev(inp["a_val"]), dev(inp["D"]),
                   carry_state=carry, workspace=ws)
    torch.cuda.synchronize()
    return host(y), host(ssm), host(kst), host(vst)


@pytest.mark.parametrize("dtype", [orc.BF16, orc.F16, orc.F32])
@pytest.mark.parametrize("shape", SSD_SHAPES)
@pytest.mark.parametrize("carry", [False, True])
@pytest.mark.parametrize("dt_scale", [1.0, 0.03])
def test_m3_ssd_matches_oracle(shape, dtype, carry, dt_scale):
    """Chunked SSD vs the f64 chunked oracle (== the sequential definition).  At 16-bit storage the
    matrix-core operands (P, w*x, the entering state) are rounded to the storage type, so the final
    state is held to the storage tolerance too; at f32 storage the recurrence kernel runs (1e-4)."""
    B, T, nh, hd, ds = shape
    rng = np.random.default_rng(hash((shape, dtype, carry)) & 0xFFFF)
    inp = quantised(rng, B, T, nh, hd, ds, dtype, dt_scale)
    st0 = rand_state(rng, B, nh, hd, ds, dtype, zero=False)
    print(f"case m3 ssd shape={shape} dtype={dtype} carry={carry} dt_scale={dt_scale}", flush=True)
    y_ref, s_ref, k_ref, v_ref = orc.m3_chunked_f64(*st0, inp["x"], inp["K"], inp["Q"], inp["dt"], inp["trap"], inp["a_val"],
                                                    inp["D"], 64, carry=carry)
    y, ssm, kst, vst = run_ssd(inp, st0, dtype, carry)
    assert_close(y, y_ref, dtype, "y")
    assert_close(ssm, s_ref, dtype, "ssm")
    assert np.array_equal(kst, k_ref.astype(np.float32)) and np.array_equal(vst, v_ref.astype(np.float32))


@pytest.mark.parametrize("carry", [False, True])
def test_m3_ssd_super_chunk_split_matches_single_walk(carry):
    """With a workspace the sequence is cut into super-chunks that run concurrently; without one a single
    workgroup walks all chunks.  Same operands, same matrix-core rounding: the two must agree far inside the
    storage tolerance (only the f32 summation order of the entering state differs)."""
    B, T, nh, hd, ds = 1, 1500, 2, 64, 32
    rng = np.random.default_rng(77)
    inp = quantised(rng, B, T, nh, hd, ds, orc.BF16, 0.03)
    st0 = rand_state(rng, B, nh, hd, ds, orc.BF16)
    print(f"case m3 ssd split-vs-walk carry={carry}", flush=True)
    y1, s1, k1, v1 = run_ssd(inp, st0, orc.BF16, carry, use_ws=True)
    y2, s2, k2, v2 = run_ssd(inp, st0, orc.BF16, carry, use_ws=False)
    assert_close(y1, y2, orc.BF16, "y split vs walk")
    assert np.allclose(s1, s2, rtol=1e-3, atol=1e-3 * np.abs(s2).max())
    assert np.array_equal(k1, k2) and np.array_equal(v1, v2)


def test_m3_ssd_full_size_vs_sequential_kernel_and_oracle_subset():
    """The Mamba-3 prefill workload (batch 4 x T 4096, 24 heads, headdim 64, d_state 64, bf16): the chunked
    matrix-core kernel against (a) the oracle on two heads (heads are independent) and (b) the sequential
    recurrence kernel on every head -- the chunked == sequential identity at full size."""
    B, T, nh, hd, ds = 4, 4096, 24, 64, 64
    rng = np.random.default_rng(12)
    inp = quantised(rng, B, T, nh, hd, ds, orc.BF16)
    z = rand_state(rng, B, nh, hd, ds, orc.BF16, zero=True)
    y, ssm, kst, vst = run_ssd(inp, z, orc.BF16, False)
    sel = [3, 17]
    sub = dict(x=inp["x"].reshape(B, T, nh, hd)[:, :, sel].reshape(B, T, len(sel) * hd), K=inp["K"][:, :, sel], Q=inp["Q"][:, :, sel],
               dt=inp["dt"][:, :, sel], trap=inp["trap"][:, :, sel], a_val=inp["a_val"][:, :, sel], D=inp["D"][sel])
    zs = (np.zeros((B, 2, hd, ds)), np.zeros((B, 2, ds)), np.zeros((B, 2, hd)))
    y_ref, s_ref, _, _ = orc.m3_chunked_f64(*zs, sub["x"], sub["K"], sub["Q"], sub["dt"], sub["trap"], sub["a_val"], sub["D"], 64)
    assert_close(y.reshape(B, T, nh, hd)[:, :, sel].reshape(B, T, 2 * hd), y_ref, orc.BF16, "y[2 heads]")
    assert_close(ssm[:, sel], s_ref, orc.BF16, "ssm[2 heads]")
    # sequential kernel over everything
    al, be, ga = ops.m3_compute_abg(dev(inp["dt"]), dev(inp["a_val"]), dev(inp["trap"]))
    s2, k2, v2 = (dev(s) for s in z)
    x = dev(inp["x"], orc.BF16)
    y2 = torch.empty_like(x)
    ops.m3_seq_fwd(s2, k2, v2, y2, x, dev(inp["K"], orc.BF16), dev(inp["Q"], orc.BF16), al, be, ga, dev(inp["D"]))
    assert cosine(y, host(y2)) >= 0.9999 and cosine(ssm, host(s2)) >= 0.9999
    assert np.array_equal(kst, host(k2)) and np.array_equal(vst, host(v2))


def test_m3_rejects_bad_arguments():
    from mamba_rs_amd import MambaHipError
    rng = np.random.default_rng(1)
    inp = quantised(rng, 1, 8, 2, 16, 16, orc.BF16)
    st0 = rand_state(rng, 1, 2, 16, 16, orc.BF16)
    x, K, Q = dev(inp["x"], orc.BF16), dev(inp["K"], orc.BF16), dev(inp["Q"], orc.BF16)
    ssm, kst, vst = (dev(s) for s in st0)
    y = torch.empty_like(x)
    with pytest.raises(MambaHipError) as e:   # chunk size other than 64
        ops.m3_ssd_fwd(ssm, kst, vst, y, x, K, Q, dev(inp["dt"]), dev(inp["trap"]), dev(inp["a_val"]), dev(inp["D"]), chunk_size=32)
    assert e.value.code == -2
    x48 = torch.zeros(1, 8, 2 * 48, device=DEV, dtype=torch.bfloat16)  # headdim 48: not a matrix-core shape
    with pytest.raises(MambaHipError) as e:
        ops.m3_ssd_fwd(torch.zeros(1, 2, 48, 16, device=DEV), kst, torch.zeros(1, 2, 48, device=DEV), torch.empty_like(x48), x48, K, Q,
                       dev(inp["dt"]), dev(inp["trap"]), dev(inp["a_val"]), dev(inp["D"]))
    assert e.value.code == -2
    # tiles move as 16-byte row pieces: an output that starts 2 bytes off a 16-byte boundary is refused, not written
    y_off = torch.empty(x.numel() + 8, device=DEV, dtype=torch.bfloat16)[1:1 + x.numel()].view(x.shape)
    with pytest.raises(MambaHipError) as e:
        ops.m3_ssd_fwd(ssm, kst, vst, y_off, x, K, Q, dev(inp["dt"]), dev(inp["trap"]), dev(inp["a_val"]), dev(inp["D"]))
    assert e.value.code == -5
