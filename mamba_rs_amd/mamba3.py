"""Mamba-3 SISO host mirror: Mamba3Config, Mamba3Weights and GpuMamba3Backbone
(src/mamba3_siso/{config,weights}.rs, src/mamba3_siso/gpu/inference.rs:1487-1671) over the C ABI.

All arithmetic happens in libmamba_hip.so; this module marshals numpy arrays and restates the
reference's deterministic initialiser so that synthetic models can be built without it.
"""
from __future__ import annotations

import math
from ctypes import POINTER, Structure, byref, c_float, c_int, c_void_p
from dataclasses import dataclass, field

import numpy as np

from . import _lib
from .config import WeightDtype

_FP = POINTER(c_float)


@dataclass
class Mamba3Config:
    """src/mamba3_siso/config.rs:7-58 (defaults :133-147)."""
    d_model: int = 128
    d_state: int = 16
    expand: int = 2
    headdim: int = 16
    ngroups: int = 1
    n_layers: int = 3
    rope_fraction: float = 0.5
    a_floor: float = 1e-4
    is_outproj_norm: bool = False
    rms_norm_eps: float = 1e-5

    def d_inner(self) -> int:
        return self.d_model * self.expand

    def nheads(self) -> int:
        return self.d_inner() // self.headdim

    def num_rope_angles(self) -> int:
        # floor(d_state * rope_fraction) / 2, evaluated in f32 as the reference does (config.rs:45-47)
        return int(np.float32(self.d_state) * np.float32(self.rope_fraction)) // 2

    def in_proj_out_dim(self) -> int:
        return 2 * self.d_inner() + 2 * self.ngroups * self.d_state + 3 * self.nheads() + self.num_rope_angles()

    def validate(self) -> None:
        """config.rs:66-131, with this library's limits in place of headdim <= 32 / d_state <= 64."""
        for n in ("d_model", "d_state", "expand", "headdim", "ngroups", "n_layers"):
            if getattr(self, n) < 1:
                raise ValueError(f"{n} must be > 0")
        if self.d_inner() % self.headdim:
            raise ValueError("d_inner must be a multiple of headdim")
        if self.nheads() % self.ngroups:
            raise ValueError("nheads must be a multiple of ngroups")
        lg = self.d_state // 4
        if self.d_state % 4 or lg & (lg - 1) or lg > 64 or self.headdim * lg > 1024 or (self.headdim * lg) % 64:
            raise ValueError("d_state must be 4 x a power of two <= 256 and headdim * d_state / 4 a multiple of 64 <= 1024")
        if not (self.rope_fraction == 0.5 or self.rope_fraction == 1.0):
            raise ValueError("rope_fraction must be 0.5 or 1.0")
        if not self.a_floor > 0:
            raise ValueError("a_floor must be > 0")


_LAYER_FIELDS = ("norm_weight", "in_proj_w", "dt_bias", "b_norm_weight", "c_norm_weight", "b_bias", "c_bias", "d_param",
                 "norm_gate_weight", "out_proj_w")


@dataclass
class Mamba3LayerWeights:
    norm_weight: np.ndarray
    in_proj_w: np.ndarray
    dt_bias: np.ndarray
    b_norm_weight: np.ndarray
    c_norm_weight: np.ndarray
    b_bias: np.ndarray
    c_bias: np.ndarray
    d_param: np.ndarray
    norm_gate_weight: np.ndarray
    out_proj_w: np.ndarray


def _xorshift64_f32(state: int, n: int):
    """n draws of the reference's xorshift64 (13, 7, 17) mapped to [0, 1) by the low 24 bits (weights.rs:51-65)."""
    out = np.empty(n, np.float32)
    m = (1 << 64) - 1
    s = state
    for i in range(n):
        s ^= (s << 13) & m
        s ^= s >> 7
        s ^= (s << 17) & m
        out[i] = np.float32(s & 0xFFFFFF) / np.float32(16777216.0)
    return out, s


@dataclass
class Mamba3Weights:
    input_proj_w: np.ndarray
    input_proj_b: np.ndarray
    layers: list = field(default_factory=list)
    norm_f_weight: np.ndarray = None

    @classmethod
    def init(cls, cfg: Mamba3Config, input_dim: int, seed: int) -> "Mamba3Weights":
        """Mamba3Weights::init (weights.rs:120-147): Kaiming-uniform projections in draw order input_proj, then per
        layer in_proj, out_proj, dt_bias = inv_softplus(log-uniform[1e-3, 1e-1]); B/C bias, norms and D are ones."""
        cfg.validate()
        dm, ds, di, nh, ip = cfg.d_model, cfg.d_state, cfg.d_inner(), cfg.nheads(), cfg.in_proj_out_dim()
        s = max(int(seed), 1)

        def kaiming(n, fan_in):
            nonlocal s
            u, s = _xorshift64_f32(s, n)
            bound = np.float32(math.sqrt(3.0 / fan_in))
            return (u * np.float32(2.0) - np.float32(1.0)) * bound

        ipw = kaiming(input_dim * dm, input_dim).reshape(input_dim, dm)
        layers = []
        # f32 libm calls evaluated through f64 and rounded once (what a correctly rounded expf/logf returns); the
        # subtraction exp(dt) - 1 stays in f32 as in the reference (weights.rs:134-139)
        f32 = lambda v: np.asarray(v, dtype=np.float64).astype(np.float32)
        lmin, lmax = f32(np.log(np.float64(np.float32(0.001)))), f32(np.log(np.float64(np.float32(0.1))))
        for _ in range(cfg.n_layers):
            inw = kaiming(dm * ip, dm).reshape(dm, ip)
            outw = kaiming(di * dm, di).reshape(di, dm)
            u, s = _xorshift64_f32(s, nh)
            dtv = f32(np.exp((u * (lmax - lmin) + lmin).astype(np.float64)))
            inv = f32(np.log((f32(np.exp(dtv.astype(np.float64))) - np.float32(1.0)).astype(np.float64)))
            dtb = np.where(dtv > 20.0, dtv, inv).astype(np.float32)
            layers.append(Mamba3LayerWeights(np.ones(dm, np.float32), inw, dtb, np.ones(ds, np.float32), np.ones(ds, np.float32),
                                             np.ones((nh, ds), np.float32), np.ones((nh, ds), np.float32), np.ones(nh, np.float32),
                                             np.ones(di, np.float32), outw))
        return cls(ipw, np.zeros(dm, np.float32), layers, np.ones(dm, np.float32))

    @classmethod
    def random_lm(cls, cfg: Mamba3Config, seed: int, std: float = 0.02) -> "Mamba3Weights":
        """Random-init weights of an LM-shaped backbone (identity input_proj) drawn with numpy's generator -- for
        benchmarks at sizes where the reference's sequential xorshift initialiser (`init`) would take minutes in
        Python: projections N(0, std), dt bias inv_softplus(log-uniform[1e-3, 1e-1]), the rest ones as in `init`."""
        cfg.validate()
        rng = np.random.default_rng(seed)
        dm, ds, di, nh, ip = cfg.d_model, cfg.d_state, cfg.d_inner(), cfg.nheads(), cfg.in_proj_out_dim()
        n = lambda *s: (rng.standard_normal(s, dtype=np.float32) * np.float32(std))
        layers = []
        for _ in range(cfg.n_layers):
            dt = np.exp(rng.uniform(np.log(1e-3), np.log(1e-1), nh))
            layers.append(Mamba3LayerWeights(np.ones(dm, np.float32), n(dm, ip), np.log(np.expm1(dt)).astype(np.float32),
                                             np.ones(ds, np.float32), np.ones(ds, np.float32), np.ones((nh, ds), np.float32),
                                             np.ones((nh, ds), np.float32), np.ones(nh, np.float32), np.ones(di, np.float32), n(di, dm)))
        return cls(np.zeros(0, np.float32), np.zeros(dm, np.float32), layers, np.ones(dm, np.float32))

    def validate(self, cfg: Mamba3Config, input_dim: int) -> None:
        dm, ds, di, nh, ip = cfg.d_model, cfg.d_state, cfg.d_inner(), cfg.nheads(), cfg.in_proj_out_dim()
        if self.input_proj_w.size not in (0, input_dim * dm):
            raise ValueError("input_proj_w must be empty (identity) or [input_dim, d_model]")
        if len(self.layers) != cfg.n_layers:
            raise ValueError("layer count mismatch")
        want = dict(norm_weight=dm, in_proj_w=dm * ip, dt_bias=nh, b_norm_weight=ds, c_norm_weight=ds, b_bias=nh * ds, c_bias=nh * ds,
                    d_param=nh, norm_gate_weight=di, out_proj_w=di * dm)
        for i, lw in enumerate(self.layers):
            for n, k in want.items():
                if getattr(lw, n).size != k:
                    raise ValueError(f"layer {i}: {n} has {getattr(lw, n).size} elements, expected {k}")
        if self.norm_f_weight.size != dm:
            raise ValueError("norm_f_weight must be [d_model]")


class _CConfig3(Structure):
    _fields_ = [("d_model", c_int), ("d_state", c_int), ("expand", c_int), ("headdim", c_int), ("ngroups", c_int), ("n_layers", c_int),
                ("n_rope_angles", c_int), ("a_floor", c_float), ("is_outproj_norm", c_int), ("rms_norm_eps", c_float)]


class _CLayer3(Structure):
    _fields_ = [(n, _FP) for n in _LAYER_FIELDS]


class _CWeights3(Structure):
    _fields_ = [("input_proj_w", _FP), ("input_proj_b", _FP), ("layers", POINTER(_CLayer3)), ("norm_f_weight", _FP)]


def _fp(a: np.ndarray):
    return a.ctypes.data_as(_FP)


def _bind():
    lib = _lib.load()
    if getattr(lib, "_m3_engine_bound", False):
        return lib
    P = c_void_p
    sigs = {
        "mrs_m3_backbone_create": (c_int, [POINTER(P), c_int, POINTER(_CWeights3), POINTER(_CConfig3), c_int, c_int, c_int]),
        "mrs_m3_backbone_destroy": (None, [P]),
        "mrs_m3_backbone_step": (c_int, [P, _FP, _FP]),
        "mrs_m3_backbone_step_gpu_only": (c_int, [P]),
        "mrs_m3_backbone_reset": (c_int, [P]),
        "mrs_m3_backbone_capture_graph": (c_int, [P]),
        "mrs_m3_backbone_temporal_ptr": (P, [P]),
        "mrs_m3_backbone_temporal_dtype": (c_int, [P]),
        "mrs_m3_backbone_decode_route": (c_int, [P]),
        "mrs_m3_backbone_input_ptr": (P, [P]),
        "mrs_m3_backbone_stream": (P, [P]),
        "mrs_m3_backbone_sync": (c_int, [P]),
        "mrs_m3_backbone_download_state": (c_int, [P, c_int, _FP, _FP, _FP, _FP]),
        "mrs_m3_backbone_alloc_prefill_scratch": (c_int, [P, c_int]),
        "mrs_m3_backbone_prefill_sequence": (c_int, [P, _FP, c_int, _FP]),
        "mrs_m3_backbone_prefill_device": (c_int, [P, c_int]),
        "mrs_m3_backbone_set_gemm_tuning": (c_int, [P, c_int]),
        "mrs_m3_backbone_prefill_input_ptr": (P, [P]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    lib._m3_engine_bound = True
    lib._m3_engine_names = sorted(sigs)
    return lib


def m3_engine_exported_names():
    return list(_bind()._m3_engine_names)


def _call(name, *args):
    lib = _bind()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise _lib.MambaHipError(name, rc, lib.mrs_last_error().decode())


class GpuMamba3Backbone:
    """One-GPU Mamba-3 SISO backbone with fixed batch: `step` advances every batch row by one token."""

    def __init__(self, gpu_ordinal: int, weights: Mamba3Weights, cfg: Mamba3Config, input_dim: int, batch: int,
                 dtype: WeightDtype = WeightDtype.F32):
        cfg.validate()
        weights.validate(cfg, input_dim)
        self.cfg, self.input_dim, self.batch, self.dtype = cfg, input_dim, batch, WeightDtype(dtype)
        keep = []

        def arr(a):
            a = np.ascontiguousarray(a, dtype=np.float32)
            keep.append(a)
            return _fp(a)

        layers = (_CLayer3 * cfg.n_layers)()
        for i, lw in enumerate(weights.layers):
            for n in _LAYER_FIELDS:
                setattr(layers[i], n, arr(getattr(lw, n)))
        cw = _CWeights3()
        identity = weights.input_proj_w.size == 0
        cw.input_proj_w = None if identity else arr(weights.input_proj_w)
        cw.input_proj_b = None if identity else arr(weights.input_proj_b)
        cw.layers = layers
        cw.norm_f_weight = arr(weights.norm_f_weight)
        cc = _CConfig3(cfg.d_model, cfg.d_state, cfg.expand, cfg.headdim, cfg.ngroups, cfg.n_layers, cfg.num_rope_angles(),
                       cfg.a_floor, 1 if cfg.is_outproj_norm else 0, cfg.rms_norm_eps)
        h = c_void_p()
        _call("mrs_m3_backbone_create", byref(h), gpu_ordinal, byref(cw), byref(cc), input_dim, batch, int(self.dtype))
        self._h = h

    @classmethod
    def new(cls, gpu_ordinal, weights, cfg, input_dim, batch):
        return cls(gpu_ordinal, weights, cfg, input_dim, batch, WeightDtype.F32)

    @classmethod
    def new_with_dtype(cls, gpu_ordinal, weights, cfg, input_dim, batch, dtype):
        return cls(gpu_ordinal, weights, cfg, input_dim, batch, dtype)

    def close(self):
        if getattr(self, "_h", None):
            _bind().mrs_m3_backbone_destroy(self._h)
            self._h = None

    __del__ = close

    def step(self, inp: np.ndarray) -> np.ndarray:
        inp = np.ascontiguousarray(inp, dtype=np.float32)
        if inp.size != self.batch * self.input_dim:
            raise ValueError(f"input must hold batch*input_dim = {self.batch * self.input_dim} values")
        out = np.empty((self.batch, self.cfg.d_model), np.float32)
        _call("mrs_m3_backbone_step", self._h, _fp(inp), _fp(out))
        return out

    def step_gpu_only(self):
        _call("mrs_m3_backbone_step_gpu_only", self._h)

    def alloc_prefill_scratch(self, T: int):
        _call("mrs_m3_backbone_alloc_prefill_scratch", self._h, T)

    def prefill_sequence(self, inp: np.ndarray) -> np.ndarray:
        """inp [batch, T, input_dim] f32 -> norm_f output of the last position [batch, d_model]; the state is left
        positioned for step()."""
        inp = np.ascontiguousarray(inp, dtype=np.float32)
        if inp.ndim != 3 or inp.shape[0] != self.batch or inp.shape[2] != self.input_dim:
            raise ValueError("input must be [batch, T, input_dim]")
        out = np.empty((self.batch, self.cfg.d_model), np.float32)
        _call("mrs_m3_backbone_prefill_sequence", self._h, _fp(inp), inp.shape[1], _fp(out))
        return out

    def prefill_device(self, T: int):
        _call("mrs_m3_backbone_prefill_device", self._h, T)

    def prefill_input_ptr(self) -> int:
        return _bind().mrs_m3_backbone_prefill_input_ptr(self._h)

    def reset(self):
        _call("mrs_m3_backbone_reset", self._h)

    def capture_graph(self):
        _call("mrs_m3_backbone_capture_graph", self._h)

    def sync(self):
        _call("mrs_m3_backbone_sync", self._h)

    def set_gemm_tuning(self, on: bool = True):
        """Time the GEMM library's kernels for each prefill projection shape once and keep the fastest."""
        _call("mrs_m3_backbone_set_gemm_tuning", self._h, 1 if on else 0)

    def temporal_ptr(self) -> int:
        return _bind().mrs_m3_backbone_temporal_ptr(self._h)

    def temporal_dtype(self) -> WeightDtype:
        return WeightDtype(_bind().mrs_m3_backbone_temporal_dtype(self._h))

    def decode_route(self) -> int:
        """0: chain on the vendor GEMM, 1: the library's own fused chain, 2: a whole step in one launch."""
        return _bind().mrs_m3_backbone_decode_route(self._h)

    def input_ptr(self) -> int:
        return _bind().mrs_m3_backbone_input_ptr(self._h)

    def stream(self) -> int:
        return _bind().mrs_m3_backbone_stream(self._h)

    def download_state(self, layer: int):
        c, B = self.cfg, self.batch
        nh, na = c.nheads(), max(c.num_rope_angles(), 1)
        ssm = np.empty((B, nh, c.headdim, c.d_state), np.float32)
        k = np.empty((B, nh, c.d_state), np.float32)
        v = np.empty((B, nh, c.headdim), np.float32)
        ang = np.empty((B, nh, na), np.float32)
        _call("mrs_m3_backbone_download_state", self._h, layer, _fp(ssm), _fp(k), _fp(v), _fp(ang))
        return ssm, k, v, ang
