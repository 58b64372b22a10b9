"""MambaWeights: the reference's flat f32 weight container and its seeded initialiser.

Layout and draw order follow src/weights.rs:7-161, 224-250: linear weights are row-major
[n_in, n_out]; the LCG  s <- s*6364136223846793005 + 1442695040888963407 (mod 2^64),
f = (s >> 40) / 2^24  is drawn for input_proj, then per layer in_proj, conv1d, x_proj, dt_proj,
dt_proj bias, out_proj.  The stream is generated in closed form (vectorised), bit-identical to
the sequential recurrence.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from .config import MambaConfig

_A = np.uint64(6364136223846793005)
_C = np.uint64(1442695040888963407)


class _Lcg:
    """SimpleRng of src/weights.rs:224-239, drawn in blocks."""

    def __init__(self, seed: int):
        self.s = np.uint64(seed & 0xFFFFFFFFFFFFFFFF)

    def next_f32(self, n: int) -> np.ndarray:
        if n == 0:
            return np.zeros(0, np.float32)
        with np.errstate(over="ignore"):
            a = np.full(n, _A, dtype=np.uint64)
            apow = np.multiply.accumulate(a)                       # A^1 .. A^n (mod 2^64)
            geo = np.empty(n, dtype=np.uint64)                     # sum_{j<k} A^j, k = 1..n
            geo[0] = np.uint64(1)
            if n > 1:
                geo[1:] = np.add.accumulate(apow[:-1]) + np.uint64(1)
            states = apow * self.s + _C * geo
        self.s = states[-1]
        return (states >> np.uint64(40)).astype(np.float32) / np.float32(1 << 24)


@dataclass
class MambaLayerWeights:
    norm_weight: np.ndarray
    in_proj_w: np.ndarray
    conv1d_weight: np.ndarray
    conv1d_bias: np.ndarray
    x_proj_w: np.ndarray
    dt_proj_w: np.ndarray
    dt_proj_b: np.ndarray
    a_log: np.ndarray
    d_param: np.ndarray
    out_proj_w: np.ndarray

    def a_neg(self) -> np.ndarray:
        """compute_a_neg (src/weights.rs:44-48)."""
        return -np.exp(self.a_log)


@dataclass
class MambaWeights:
    input_proj_w: np.ndarray            # [input_dim, d_model]; size 0 = identity (LM / HF case)
    input_proj_b: np.ndarray
    layers: list = field(default_factory=list)
    norm_f_weight: np.ndarray = None

    @staticmethod
    def zeros(cfg: MambaConfig, input_dim: int) -> "MambaWeights":
        d, di, ds, dc, dr, xd = cfg.d_model, cfg.d_inner(), cfg.d_state, cfg.d_conv, cfg.dt_rank(), cfg.xdbl_dim()
        f = np.float32
        layers = [MambaLayerWeights(np.ones(d, f), np.zeros((d, 2 * di), f), np.zeros((di, dc), f), np.zeros(di, f),
                                    np.zeros((di, xd), f), np.zeros((dr, di), f), np.zeros(di, f), np.zeros((di, ds), f),
                                    np.ones(di, f), np.zeros((di, d), f)) for _ in range(cfg.n_layers)]
        return MambaWeights(np.zeros((input_dim, d), f), np.zeros(d, f), layers, np.ones(d, f))

    @staticmethod
    def init(cfg: MambaConfig, input_dim: int, seed: int) -> "MambaWeights":
        """MambaWeights::init (src/weights.rs:107-161)."""
        w = MambaWeights.zeros(cfg, input_dim)
        rng = _Lcg(seed)
        d, di, ds, dc, dr = cfg.d_model, cfg.d_inner(), cfg.d_state, cfg.d_conv, cfg.dt_rank()

        def kaiming(shape, fan_in):
            bound = np.sqrt(np.float32(3.0) / np.float32(fan_in))
            return (-bound + np.float32(2.0) * bound * rng.next_f32(int(np.prod(shape)))).reshape(shape).astype(np.float32)

        w.input_proj_w = kaiming((input_dim, d), input_dim)
        lmin = np.float32(np.log(np.float64(np.float32(0.001))))
        lmax = np.float32(np.log(np.float64(np.float32(0.1))))
        for lw in w.layers:
            lw.in_proj_w = kaiming((d, 2 * di), d)
            lw.conv1d_weight = kaiming((di, dc), dc)
            lw.x_proj_w = kaiming((di, cfg.xdbl_dim()), di)
            lw.dt_proj_w = kaiming((dr, di), dr)
            # f32 expf/logf evaluated as correctly rounded values (libm is within an ulp of that); the
            # subtraction exp(dt) - 1 stays in f32 as in the reference (inv_softplus, src/weights.rs:248-250)
            f32 = lambda v: np.asarray(v, dtype=np.float64).astype(np.float32)
            dt = f32(np.exp((rng.next_f32(di) * (lmax - lmin) + lmin).astype(np.float64)))
            lw.dt_proj_b = f32(np.log((f32(np.exp(dt.astype(np.float64))) - np.float32(1.0)).astype(np.float64)))
            lw.a_log = np.tile(np.log(np.arange(1, ds + 1, dtype=np.float32)), (di, 1)).astype(np.float32)
            lw.out_proj_w = kaiming((di, d), di)
        return w

    @staticmethod
    def random_lm(cfg: MambaConfig, seed: int, std: float = 0.02) -> "MambaWeights":
        """Random-init weights of an LM-shaped backbone (identity input_proj): projections N(0, std),
        conv1d Kaiming-uniform, A / dt bias / D / norms as in `init`."""
        rng = np.random.default_rng(seed)
        d, di, ds, dc, dr = cfg.d_model, cfg.d_inner(), cfg.d_state, cfg.d_conv, cfg.dt_rank()
        w = MambaWeights.zeros(cfg, 0)
        w.input_proj_w = np.zeros((0, d), np.float32)
        n = lambda *s: (rng.standard_normal(s, dtype=np.float32) * np.float32(std))
        for lw in w.layers:
            lw.in_proj_w = n(d, 2 * di)
            b = np.sqrt(3.0 / dc)
            lw.conv1d_weight = rng.uniform(-b, b, (di, dc)).astype(np.float32)
            lw.x_proj_w = n(di, cfg.xdbl_dim())
            lw.dt_proj_w = n(dr, di)
            dt = np.exp(rng.uniform(np.log(1e-3), np.log(1e-1), di))
            lw.dt_proj_b = np.log(np.expm1(dt)).astype(np.float32)
            lw.a_log = np.tile(np.log(np.arange(1, ds + 1, dtype=np.float32)), (di, 1)).astype(np.float32)
            lw.out_proj_w = n(di, d)
        return w

    def validate(self, cfg: MambaConfig, input_dim: int) -> None:
        """MambaWeights::validate (src/weights.rs:163-206); raises ValueError."""
        d, di, ds, dc, dr, xd = cfg.d_model, cfg.d_inner(), cfg.d_state, cfg.d_conv, cfg.dt_rank(), cfg.xdbl_dim()

        def check(name, arr, n):
            if arr.size != n:
                raise ValueError(f"{name}: expected {n}, got {arr.size}")

        if self.input_proj_w.size:
            check("input_proj_w", self.input_proj_w, input_dim * d)
        check("norm_f_weight", self.norm_f_weight, d)
        if len(self.layers) != cfg.n_layers:
            raise ValueError(f"expected {cfg.n_layers} layers, got {len(self.layers)}")
        for i, lw in enumerate(self.layers):
            for name, n in (("norm_weight", d), ("in_proj_w", d * 2 * di), ("conv1d_weight", di * dc), ("conv1d_bias", di),
                            ("x_proj_w", di * xd), ("dt_proj_w", dr * di), ("dt_proj_b", di), ("a_log", di * ds),
                            ("d_param", di), ("out_proj_w", di * d)):
                check(f"layer[{i}].{name}", getattr(lw, name), n)
