"""GPU: the scan entry point that allocates nothing (mrs_ssm_scan_fwd_static) against mrs_ssm_scan_fwd_ex.

Both run the same kernels on the same chunk plan, the one with its chunk summaries in the caller's workspace, the other
in the library's own per-GPU buffer, so y and the final state must be identical bit for bit -- on two calls in a row,
the second on a smaller input (the buffer then still holds the first call's summaries beyond what the second one
writes), and again for a shape that takes the serial route.  The shapes are also held to the f64 oracle."""
import numpy as np
import pytest
import torch

import orc
from gpu_util import assert_close, dev, host, quant
from util import scan_inputs

pytestmark = pytest.mark.gpu

from mamba_rs_amd import MambaHipError, ops  # noqa: E402


def run_both(rng, batch, T, di, dtype, gated, s4d=True, check_oracle=True):
    ds = 16
    inp = scan_inputs(rng, batch, T, di, ds, s4d=s4d)
    for k in ("u", "delta", "B", "C", "z"):
        inp[k] = quant(inp[k], dtype)
    h0 = (rng.standard_normal((batch, di, ds)) * 0.1).astype(np.float32)
    d = {k: dev(inp[k], dtype) for k in ("u", "delta", "B", "C", "z")}
    a_neg, D = dev(inp["a_neg"]), dev(inp["D"])
    flags = (ops.GATE_SILU if gated else 0) | (ops.A_S4D_REAL if s4d else 0)
    gate = d["z"] if gated else None
    ws = torch.empty(max(ops.ssm_scan_workspace_bytes(batch, T, di, ds), 256), dtype=torch.uint8, device="cuda:0")
    h_a, y_a = dev(h0), torch.empty_like(d["delta"])
    ops.ssm_scan_fwd(h_a, y_a, d["delta"], d["u"], d["B"], d["C"], a_neg, D, gate=gate, flags=flags, workspace=ws)
    h_b, y_b = dev(h0), torch.empty_like(d["delta"])
    ops.ssm_scan_fwd(h_b, y_b, d["delta"], d["u"], d["B"], d["C"], a_neg, D, gate=gate, flags=flags, static_scratch=True)
    torch.cuda.synchronize()
    assert torch.equal(y_a, y_b), "y differs between the workspace and the built-in buffer"
    assert torch.equal(h_a, h_b), "final state differs between the workspace and the built-in buffer"
    if check_oracle:
        y_ref, h_ref = orc.m1_scan_f64(h0, inp["delta"], inp["u"], inp["B"], inp["C"], inp["a_neg"], inp["D"],
                                       gate=inp["z"] if gated else None, gate_mode=2 if gated else 0)
        assert_close(host(y_b), y_ref, dtype, "y")
        assert_close(host(h_b), h_ref, orc.F32, "h")


def test_static_scratch_scan_equals_the_workspace_scan_on_two_calls_in_a_row():
    rng = np.random.default_rng(70)
    print("case static scan: 3 x 1000 x 320 bf16 gated, then 2 x 300 x 192", flush=True)
    run_both(rng, 3, 1000, 320, orc.BF16, True)        # T-split route, ragged last chunk, partial channel tile
    free0 = torch.cuda.mem_get_info()[0]
    run_both(rng, 2, 300, 192, orc.BF16, True)         # smaller: fewer chunks, the buffer keeps stale summaries beyond them
    run_both(rng, 2, 520, 128, orc.F32, False, s4d=False)
    run_both(rng, 2, 40, 64, orc.F16, True)            # short: the serial route, which needs no buffer at all
    # nothing was allocated by the library in between (the tensors of the test itself come from torch's cached blocks
    # or are released again; a leak of the buffer's size class would show)
    torch.cuda.synchronize()
    assert abs(torch.cuda.mem_get_info()[0] - free0) < (12 << 20)


@pytest.mark.parametrize("shape", [(8, 2048, 1536), (4, 4096, 5120)])
def test_static_scratch_scan_at_the_benchmark_shapes(shape):
    rng = np.random.default_rng(71)
    print(f"case static scan: {shape} bf16 gated (bit-equality only)", flush=True)
    run_both(rng, *shape, orc.BF16, True, check_oracle=False)


def test_static_scratch_scan_refuses_shapes_beyond_its_buffer():
    need = ops.ssm_scan_workspace_bytes(40, 512, 4096, 16)
    assert need > ops.SCAN_STATIC_SCRATCH_BYTES
    t = torch.zeros(16, dtype=torch.bfloat16, device="cuda:0")
    f = torch.zeros(16, dtype=torch.float32, device="cuda:0")
    from mamba_rs_amd import _lib
    with pytest.raises(MambaHipError) as e:
        _lib.call("mrs_ssm_scan_fwd_static", None, 2, f.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 16,
                  f.data_ptr(), f.data_ptr(), None, 0, 0, 40, 512, 4096, 16)
    assert e.value.code == -4 and "built-in buffer" in e.value.message
