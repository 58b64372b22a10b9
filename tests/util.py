"""Shared test helpers: the reference tests' deterministic generator and error metrics."""
from __future__ import annotations

import numpy as np


def det(n: int, seed: int, scale: float) -> np.ndarray:
    """xorshift32 sequence used by the reference's tests (tests/prefill.rs:25-35)."""
    out = np.empty(n, dtype=np.float32)
    s = seed & 0xFFFFFFFF
    for i in range(n):
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        out[i] = np.float32((np.float32(s & 0xFFFF) / np.float32(65536.0) - np.float32(0.5)) * np.float32(scale))
    return out


def cosine(a, b) -> float:
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    na, nb = np.linalg.norm(a), np.linalg.norm(b)
    if na == 0 and nb == 0:
        return 1.0
    return float(a @ b / (na * nb))


def max_rel(a, ref, floor: float) -> float:
    """max |a-ref| / max(|ref|, floor): relative error with an absolute floor for near-zero entries."""
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(a - ref) / np.maximum(np.abs(ref), floor)))


def scaled_err(a, ref) -> float:
    """max |a-ref| / max|ref| (error relative to the tensor's scale)."""
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(a - ref)) / max(np.max(np.abs(ref)), 1e-30))


def scan_inputs(rng: np.random.Generator, batch, T, di, ds, s4d=True):
    """Synthetic selective-scan inputs shaped like the isolated-scan workload:
    u~N(0,1); delta = softplus(0.5 N(0,1) + inv_softplus(loguniform[1e-3,1e-1]));
    a_neg = -(n+1) (S4D-real) or -exp(N(0,0.5)+log(n+1)); B,C~N(0,1); D~U(0.5,1.5); z~N(0,1)."""
    u = rng.standard_normal((batch, T, di), dtype=np.float32)
    dt = np.exp(rng.uniform(np.log(1e-3), np.log(1e-1), size=di)).astype(np.float32)
    bias = np.log(np.expm1(dt)).astype(np.float32)
    raw = 0.5 * rng.standard_normal((batch, T, di), dtype=np.float32) + bias
    delta = np.log1p(np.exp(raw)).astype(np.float32)
    n1 = np.arange(1, ds + 1, dtype=np.float32)
    if s4d:
        a_neg = np.tile(-n1, (di, 1)).astype(np.float32)
    else:
        a_neg = (-np.exp(0.5 * rng.standard_normal((di, ds)) + np.log(n1))).astype(np.float32)
    Bm = rng.standard_normal((batch, T, ds), dtype=np.float32)
    Cm = rng.standard_normal((batch, T, ds), dtype=np.float32)
    D = rng.uniform(0.5, 1.5, size=di).astype(np.float32)
    z = rng.standard_normal((batch, T, di), dtype=np.float32)
    return dict(u=u, delta=delta, a_neg=a_neg, B=Bm, C=Cm, D=D, z=z)
