"""Helpers for the GPU parity tests: numpy <-> device tensors and the north-star tolerances."""
from __future__ import annotations

import numpy as np
import torch

import orc
from util import cosine, max_rel

DEV = "cuda:0"
TORCH_DT = {orc.F32: torch.float32, orc.F16: torch.float16, orc.BF16: torch.bfloat16}
DT_NAMES = {orc.F32: "f32", orc.F16: "f16", orc.BF16: "bf16"}

# Parity bar on y and the final SSM state: rel 1e-4 at f32 storage, rel 2e-2 and
# cosine >= 0.9999 at bf16/f16 storage.  "rel" is |got-ref| / max(|ref|, rms(ref)).
REL_TOL = {orc.F32: 1e-4, orc.F16: 2e-2, orc.BF16: 2e-2}
COS_TOL = 0.9999


def quant(x, dtype):
    """Round an f32 array to the storage grid so oracle and kernel see identical bits."""
    return orc.round_to(x, dtype)


def dev(x, dtype=orc.F32):
    """f32 numpy (already on the storage grid) -> device tensor of the storage dtype."""
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(DEV).to(TORCH_DT[dtype])


def host(t):
    return t.detach().to(torch.float32).cpu().numpy()


def rms(x):
    x = np.asarray(x, dtype=np.float64)
    return float(np.sqrt(np.mean(x * x))) if x.size else 0.0


def assert_close(got, ref, dtype, what=""):
    ref = np.asarray(ref, dtype=np.float64)
    got = np.asarray(got, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    floor = max(rms(ref), 1e-30)
    err = max_rel(got, ref, floor)
    cos = cosine(got, ref)
    assert err < REL_TOL[dtype], f"{what}: rel err {err:.3e} >= {REL_TOL[dtype]:.0e} ({DT_NAMES[dtype]})"
    assert cos >= COS_TOL, f"{what}: cosine {cos:.6f} < {COS_TOL}"
    return err
