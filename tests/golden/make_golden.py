"""Writes the small input/output vectors under tests/golden/ from the CPU oracle.

The reference (a Rust crate) holds no golden vectors and cannot be built or run here, so these fixtures do
not come from it: they freeze the oracle's float64 ground truth (stored as f32) on deterministic inputs (the xorshift32
sequence the reference's own tests use, tests/prefill.rs:25-35), after the oracle has been pinned by closed
forms and independent restatements (tests/test_oracle_m1.py, tests/test_oracle_m3.py).  They guard the oracle
against drift (tests/test_golden.py, CPU) and give the kernels a fixed target (GPU).

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import orc  # noqa: E402
from util import det  # noqa: E402


def m1_scan_case():
    B, T, di, ds = 1, 260, 32, 16          # T > 256: the engine's parallel-scan route
    u = det(B * T * di, 11, 2.0).reshape(B, T, di)
    delta = np.log1p(np.exp(det(B * T * di, 12, 2.0).reshape(B, T, di) - 3.0)).astype(np.float32)
    Bm = det(B * T * ds, 13, 2.0).reshape(B, T, ds)
    Cm = det(B * T * ds, 14, 2.0).reshape(B, T, ds)
    z = det(B * T * di, 15, 4.0).reshape(B, T, di)
    a_neg = np.tile(-np.arange(1, ds + 1, dtype=np.float32), (di, 1))
    D = (1.0 + det(di, 16, 1.0)).astype(np.float32)
    h0 = det(B * di * ds, 17, 0.2).reshape(B, di, ds)
    # storage grid of the strictest 16-bit type for both: every value exactly representable in bf16 AND f16
    q = lambda a: orc.round_to(orc.round_to(a, orc.BF16), orc.F16)
    u, delta, Bm, Cm, z = (q(a) for a in (u, delta, Bm, Cm, z))
    y, h = orc.m1_scan_f64(h0, delta, u, Bm, Cm, a_neg, D, gate=z, gate_mode=2)
    return dict(u=u, delta=delta, B=Bm, C=Cm, z=z, a_neg=a_neg, D=D, h0=h0, y=y.astype(np.float32), h=h.astype(np.float32))


def conv_case():
    B, T, di, dc = 2, 37, 64, 4
    q = lambda a: orc.round_to(orc.round_to(a, orc.BF16), orc.F16)
    x = q(det(B * T * di, 21, 2.0).reshape(B, T, di))
    w = det(di * dc, 22, 1.0).reshape(di, dc)
    bias = det(di, 23, 0.2)
    st0 = det(B * di * dc, 24, 2.0).reshape(B, di, dc)
    out, st = orc.conv1d_seq_f64(st0, x, w, bias)
    return dict(x=x, w=w, bias=bias, state0=st0, out=out.astype(np.float32), state=st.astype(np.float32))


def m3_case():
    B, T, nh, hd, ds = 1, 200, 1, 32, 32   # 4 chunks of 64, ragged tail
    q = lambda a: orc.round_to(orc.round_to(a, orc.BF16), orc.F16)
    x = q(det(B * T * nh * hd, 31, 2.0).reshape(B, T, nh * hd))
    K = q(1.0 + det(B * T * nh * ds, 32, 2.0).reshape(B, T, nh, ds))
    Q = q(1.0 + det(B * T * nh * ds, 33, 2.0).reshape(B, T, nh, ds))
    dt = np.log1p(np.exp(det(B * T * nh, 34, 2.0).reshape(B, T, nh) - 5.0)).astype(np.float32)   # slow decay: state passing matters
    a_val = (-1.0 - np.abs(det(B * T * nh, 35, 2.0))).reshape(B, T, nh).astype(np.float32)
    trap = (0.5 + det(B * T * nh, 36, 0.8)).reshape(B, T, nh).astype(np.float32)
    D = (1.0 + det(nh, 37, 1.0)).astype(np.float32)
    ssm0 = det(B * nh * hd * ds, 38, 0.6).reshape(B, nh, hd, ds)
    k0 = q(det(B * nh * ds, 39, 2.0).reshape(B, nh, ds))
    v0 = q(det(B * nh * hd, 40, 2.0).reshape(B, nh, hd))
    y, ssm, kst, vst = orc.m3_chunked_f64(ssm0, k0, v0, x, K, Q, dt, trap, a_val, D, 64, carry=True)
    return dict(x=x, K=K, Q=Q, dt=dt, a_val=a_val, trap=trap, D=D, ssm0=ssm0, k0=k0, v0=v0, y=y.astype(np.float32),
                ssm=ssm.astype(np.float32), kst=kst.astype(np.float32), vst=vst.astype(np.float32))


def main():
    for name, fn in (("m1_scan", m1_scan_case), ("conv1d", conv_case), ("m3_ssd", m3_case)):
        case = fn()
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **case)
        print(name, {k: v.shape for k, v in case.items()}, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
