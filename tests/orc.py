"""numpy front end of the CPU oracle (oracle/libmamba_oracle.so). Tests only."""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_double, c_float, c_int, c_int64, c_uint64, c_void_p

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "libmamba_oracle.so")

F32, F16, BF16 = 0, 1, 2
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.run(["make", "-C", ORACLE_DIR], check=True, stdout=subprocess.DEVNULL)
        _lib = ctypes.CDLL(LIB)
        _lib.orc_fast_exp.restype = c_float
        _lib.orc_fast_exp.argtypes = [c_float]
        for n in ("orc_round_bf16", "orc_round_f16", "orc_cpu_silu", "orc_cpu_softplus", "orc_gpu_silu", "orc_gpu_softplus"):
            getattr(_lib, n).restype = c_float
            getattr(_lib, n).argtypes = [c_float]
        _lib.orc_m1_param_count.restype = c_int64
        _lib.orc_m1_layer_param_count.restype = c_int64
        _lib.orc_m1_step_scratch_len.restype = c_int64
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


def _c(a, dt=np.float32):
    return None if a is None else np.ascontiguousarray(a, dtype=dt)


def round_to(x, dtype):
    """Round an f32 array to the storage dtype's grid (RNE), returned as f32."""
    x = np.array(x, dtype=np.float32, copy=True, order="C")
    lib().orc_round_array(_p(x), c_int64(x.size), c_int(dtype))
    return x


def fast_exp(x):
    return np.array([lib().orc_fast_exp(float(v)) for v in np.asarray(x, dtype=np.float32).ravel()],
                    dtype=np.float32).reshape(np.shape(x))


def scan_use_parallel(mode, T, ds):
    return bool(lib().orc_scan_use_parallel(c_int(mode), c_int64(T), c_int64(ds)))


def _bc(Bm, Cm):
    """B and C as one contiguous buffer + stride so views into xdbl can be passed as-is."""
    Bm = _c(Bm); Cm = _c(Cm)
    return Bm, Cm, Bm.shape[-1]


def m1_scan_f64(h0, delta, u, Bm, Cm, a_neg, D, gate=None, gate_mode=0):
    """Ground truth. Returns (y f64 [B,T,di], h f64 [B,di,ds])."""
    delta = _c(delta); u = _c(u); a_neg = _c(a_neg); D = _c(D); gate = _c(gate)
    Bm, Cm, bcs = _bc(Bm, Cm)
    batch, T, di = delta.shape
    ds = a_neg.shape[1]
    h = np.array(h0, dtype=np.float64, copy=True, order="C")
    y = np.zeros((batch, T, di), dtype=np.float64)
    lib().orc_m1_scan_f64(_p(h), _p(y), _p(delta), _p(u), _p(Bm), _p(Cm), c_int64(bcs), _p(a_neg), _p(D), _p(gate),
                          c_int(gate_mode), c_int64(batch), c_int64(T), c_int64(di), c_int64(ds))
    return y, h


def m1_scan_cpu(h0, delta, u, Bm, Cm, a_neg, D, gate=None, gate_mode=0, threads=0):
    delta = _c(delta); u = _c(u); a_neg = _c(a_neg); D = _c(D); gate = _c(gate)
    Bm, Cm, bcs = _bc(Bm, Cm)
    batch, T, di = delta.shape
    ds = a_neg.shape[1]
    h = np.array(h0, dtype=np.float32, copy=True, order="C")
    y = np.zeros((batch, T, di), dtype=np.float32)
    lib().orc_m1_scan_cpu(_p(h), _p(y), _p(delta), _p(u), _p(Bm), _p(Cm), c_int64(bcs), _p(a_neg), _p(D), _p(gate),
                          c_int(gate_mode), c_int64(batch), c_int64(T), c_int64(di), c_int64(ds), c_int(threads))
    return y, h


def m1_scan_gpu(h0, delta, u, Bm, Cm, a_neg, D, gate=None, gate_mode=0, dtype=F32):
    delta = _c(delta); u = _c(u); a_neg = _c(a_neg); D = _c(D); gate = _c(gate)
    Bm, Cm, bcs = _bc(Bm, Cm)
    batch, T, di = delta.shape
    ds = a_neg.shape[1]
    h = np.array(h0, dtype=np.float32, copy=True, order="C")
    y = np.zeros((batch, T, di), dtype=np.float32)
    lib().orc_m1_scan_gpu(_p(h), _p(y), _p(delta), _p(u), _p(Bm), _p(Cm), c_int64(bcs), _p(a_neg), _p(D), _p(gate),
                          c_int(gate_mode), c_int64(batch), c_int64(T), c_int64(di), c_int64(ds), c_int(dtype))
    return y, h


def conv1d_seq_f64(state0, x, w, bias, silu=True):
    """x [B,T,di] f32; state0 [B,di,dc]. Returns (out f64, state f64)."""
    x = _c(x); w = _c(w); bias = _c(bias)
    batch, T, di = x.shape
    dc = w.shape[1]
    st = np.array(state0, dtype=np.float64, copy=True, order="C")
    out = np.zeros((batch, T, di), dtype=np.float64)
    lib().orc_conv1d_seq_silu_f64(_p(out), _p(st), _p(x), c_int64(di), _p(w), _p(bias), c_int64(batch), c_int64(T),
                                  c_int64(di), c_int64(dc), c_int(1 if silu else 0))
    return out, st


def conv1d_seq_gpu(state0, x, w, bias, silu=True, dtype=F32):
    x = _c(x); w = _c(w); bias = _c(bias)
    batch, T, di = x.shape
    dc = w.shape[1]
    st = np.array(state0, dtype=np.float32, copy=True, order="C")
    out = np.zeros((batch, T, di), dtype=np.float32)
    lib().orc_conv1d_seq_silu_gpu(_p(out), _p(st), _p(x), c_int64(di), _p(w), _p(bias), c_int64(batch), c_int64(T),
                                  c_int64(di), c_int64(dc), c_int(1 if silu else 0), c_int(dtype))
    return out, st


def conv1d_step_cpu(x, hist, w, bias):
    """CPU route: x [di] -> silu(conv), hist [di, dc-1] updated. Returns (u, hist)."""
    x = np.array(x, dtype=np.float32, copy=True, order="C")
    hist = np.array(hist, dtype=np.float32, copy=True, order="C")
    w = _c(w); bias = _c(bias)
    di, dc = w.shape
    lib().orc_conv1d_step_cpu(_p(x), _p(hist), _p(w), _p(bias), c_int64(di), c_int64(dc))
    return x, hist


def gemm(x, w, bias=None):
    x = _c(x); w = _c(w); bias = _c(bias)
    m, n_in = x.shape
    n_out = w.shape[1]
    y = np.zeros((m, n_out), dtype=np.float32)
    lib().orc_gemm(_p(y), _p(x), _p(w), _p(bias), c_int64(m), c_int64(n_in), c_int64(n_out))
    return y


def rmsnorm_rows(x, w, eps):
    x = _c(x); w = _c(w)
    out = np.zeros_like(x)
    lib().orc_rmsnorm_rows(_p(out), _p(x), _p(w), c_float(eps), c_int64(x.shape[0]), c_int64(x.shape[1]))
    return out


class M1Params:
    """Flat parameter block of MambaWeights::init with named views."""

    def __init__(self, dm, ds, dc, expand, n_layers, input_dim, seed=None, flat=None):
        self.dm, self.ds, self.dc, self.expand, self.n_layers, self.input_dim = dm, ds, dc, expand, n_layers, input_dim
        self.di = expand * dm
        self.dr = -(-dm // 16)
        self.xd = self.dr + 2 * ds
        n = lib().orc_m1_param_count(c_int64(dm), c_int64(ds), c_int64(dc), c_int64(expand), c_int64(n_layers), c_int64(input_dim))
        if flat is None:
            flat = np.zeros(n, dtype=np.float32)
            lib().orc_m1_weights_init(_p(flat), c_int64(dm), c_int64(ds), c_int64(dc), c_int64(expand), c_int64(n_layers),
                                      c_int64(input_dim), c_uint64(seed))
        assert flat.size == n
        self.flat = flat
        o = 0

        def take(*shape):
            nonlocal o
            k = int(np.prod(shape))
            v = flat[o:o + k].reshape(shape)
            o += k
            return v

        di, dr, xd = self.di, self.dr, self.xd
        self.input_proj_w = take(input_dim, dm)
        self.input_proj_b = take(dm)
        self.layers = []
        for _ in range(n_layers):
            L = dict(norm_weight=take(dm), in_proj_w=take(dm, 2 * di), conv1d_weight=take(di, dc), conv1d_bias=take(di),
                     x_proj_w=take(di, xd), dt_proj_w=take(dr, di), dt_proj_b=take(di), a_log=take(di, ds),
                     a_neg=take(di, ds), d_param=take(di), out_proj_w=take(di, dm))
            self.layers.append(L)
        self.norm_f_weight = take(dm)
        assert o == n


def m1_backbone_step(P: M1Params, x, conv_state, ssm_state, identity_proj=False, eps=1e-5):
    """One token. conv_state [L, di*(dc-1)], ssm_state [L, di*ds] are updated in place (f32 arrays)."""
    x = _c(x)
    out = np.zeros(P.dm, dtype=np.float32)
    lib().orc_m1_backbone_step(_p(out), _p(x), _p(P.flat), _p(conv_state), _p(ssm_state), c_int64(P.dm), c_int64(P.ds),
                               c_int64(P.dc), c_int64(P.expand), c_int64(P.n_layers), c_int64(P.input_dim),
                               c_int(1 if identity_proj else 0), c_float(eps))
    return out


def m1_backbone_prefill(P: M1Params, x, conv_state, ssm_state, identity_proj=False, eps=1e-5, threads=0):
    """One sequence x [T, input_dim] -> [T, dm]; state arrays updated in place."""
    x = _c(x)
    T = x.shape[0]
    out = np.zeros((T, P.dm), dtype=np.float32)
    lib().orc_m1_backbone_prefill(_p(out), _p(x), _p(P.flat), _p(conv_state), _p(ssm_state), c_int64(T), c_int64(P.dm),
                                  c_int64(P.ds), c_int64(P.dc), c_int64(P.expand), c_int64(P.n_layers),
                                  c_int64(P.input_dim), c_int(1 if identity_proj else 0), c_float(eps), c_int(threads))
    return out


def m1_zero_state(P: M1Params):
    return (np.zeros((P.n_layers, P.di * (P.dc - 1)), dtype=np.float32),
            np.zeros((P.n_layers, P.di * P.ds), dtype=np.float32))


def num_threads():
    return int(lib().orc_num_threads())


# ----------------------------------------------------------------------------- Mamba-3
def m3_abg_f64(dt, a_val, trap):
    dt = _c(dt); a_val = _c(a_val); trap = _c(trap)
    al = np.zeros(dt.shape, np.float64); be = np.zeros_like(al); ga = np.zeros_like(al)
    lib().orc_m3_abg_f64(_p(al), _p(be), _p(ga), _p(dt), _p(a_val), _p(trap), c_int64(dt.size))
    return al, be, ga


def m3_seq_f64(ssm, kst, vst, x, k, q, alpha, beta, gamma, D):
    """Sequential trapezoid in f64. x [B,T,nh*hd]; k,q [B,T,nh,ds]; alpha.. [B,T,nh] (any float dtype).
    Returns (y, ssm, kst, vst) as new f64 arrays."""
    x = _c(x); k = _c(k); q = _c(q); D = _c(D)
    al = _c(alpha, np.float64); be = _c(beta, np.float64); ga = _c(gamma, np.float64)
    B, T, nh, ds = k.shape
    hd = x.shape[2] // nh
    ssm = np.array(ssm, np.float64, copy=True, order="C"); kst = np.array(kst, np.float64, copy=True, order="C")
    vst = np.array(vst, np.float64, copy=True, order="C")
    y = np.zeros(x.shape, np.float64)
    lib().orc_m3_seq_f64(_p(ssm), _p(kst), _p(vst), _p(y), _p(x), _p(k), _p(q), _p(al), _p(be), _p(ga), _p(D),
                         c_int64(B), c_int64(T), c_int64(nh), c_int64(hd), c_int64(ds))
    return y, ssm, kst, vst


def m3_seq_gpu(ssm, kst, vst, x, k, q, alpha, beta, gamma, D, dtype=F32):
    x = _c(x); k = _c(k); q = _c(q); D = _c(D); al = _c(alpha); be = _c(beta); ga = _c(gamma)
    B, T, nh, ds = k.shape
    hd = x.shape[2] // nh
    ssm = np.array(ssm, np.float32, copy=True, order="C"); kst = np.array(kst, np.float32, copy=True, order="C")
    vst = np.array(vst, np.float32, copy=True, order="C")
    y = np.zeros(x.shape, np.float32)
    lib().orc_m3_seq_gpu(_p(ssm), _p(kst), _p(vst), _p(y), _p(x), _p(k), _p(q), _p(al), _p(be), _p(ga), _p(D),
                         c_int64(B), c_int64(T), c_int64(nh), c_int64(hd), c_int64(ds), c_int(dtype))
    return y, ssm, kst, vst


def m3_chunked_f64(ssm, kst, vst, x, K, Q, dt, trap, a_val, D, chunk, carry=False):
    x = _c(x); K = _c(K); Q = _c(Q); dt = _c(dt); trap = _c(trap); a_val = _c(a_val); D = _c(D)
    B, T, nh, ds = K.shape
    hd = x.shape[2] // nh
    ssm = np.array(ssm, np.float64, copy=True, order="C"); kst = np.array(kst, np.float64, copy=True, order="C")
    vst = np.array(vst, np.float64, copy=True, order="C")
    y = np.zeros(x.shape, np.float64)
    lib().orc_m3_chunked_f64(_p(ssm), _p(kst), _p(vst), _p(y), _p(x), _p(K), _p(Q), _p(dt), _p(trap), _p(a_val), _p(D),
                             c_int64(B), c_int64(T), c_int64(nh), c_int64(hd), c_int64(ds), c_int64(chunk),
                             c_int(1 if carry else 0))
    return y, ssm, kst, vst


class M3Params:
    """Flat parameter block of Mamba3Weights::init with named views."""

    def __init__(self, dm, ds, expand, hd, ng, n_layers, rope_fraction, input_dim, seed=None, a_floor=1e-4,
                 outproj_norm=False):
        self.dm, self.ds, self.expand, self.hd, self.ng, self.n_layers = dm, ds, expand, hd, ng, n_layers
        self.input_dim, self.a_floor, self.outproj_norm = input_dim, a_floor, outproj_norm
        self.di = dm * expand
        self.nh = self.di // hd
        self.n_rope = int(np.float32(ds) * np.float32(rope_fraction)) // 2
        self.ip = 2 * self.di + 2 * ng * ds + 3 * self.nh + self.n_rope
        L = lib()
        L.orc_m3_param_count.restype = c_int64
        n = L.orc_m3_param_count(c_int64(dm), c_int64(ds), c_int64(expand), c_int64(hd), c_int64(ng), c_int64(n_layers),
                                 c_int64(self.n_rope), c_int64(input_dim))
        flat = np.zeros(n, np.float32)
        L.orc_m3_weights_init(_p(flat), c_int64(dm), c_int64(ds), c_int64(expand), c_int64(hd), c_int64(ng),
                              c_int64(n_layers), c_int64(self.n_rope), c_int64(input_dim), c_uint64(seed))
        self.flat = flat
        o = 0

        def take(*shape):
            nonlocal o
            k = int(np.prod(shape))
            v = flat[o:o + k].reshape(shape)
            o += k
            return v

        di, nh = self.di, self.nh
        self.input_proj_w = take(input_dim, dm); self.input_proj_b = take(dm)
        self.layers = []
        for _ in range(n_layers):
            self.layers.append(dict(norm_weight=take(dm), in_proj_w=take(dm, self.ip), dt_bias=take(nh), b_norm_weight=take(ds),
                                    c_norm_weight=take(ds), b_bias=take(nh, ds), c_bias=take(nh, ds), d_param=take(nh),
                                    norm_gate_weight=take(di), out_proj_w=take(di, dm)))
        self.norm_f_weight = take(dm)
        assert o == n

    def zero_state(self):
        L, nh, hd, ds = self.n_layers, self.nh, self.hd, self.ds
        return (np.zeros((L, nh, hd, ds), np.float32), np.zeros((L, nh, ds), np.float32), np.zeros((L, nh, hd), np.float32),
                np.zeros((L, nh, max(self.n_rope, 1)), np.float32))


def m3_backbone_step(P: M3Params, x, state, taps=False):
    """One token through the Mamba-3 backbone (CPU route). state = (ssm, kst, vst, angle), updated in place.
    With taps=True also returns per-layer dict of the scan-level quantities."""
    ssm, kst, vst, angle = state
    x = _c(x)
    out = np.zeros(P.dm, np.float32)
    tp = np.zeros((P.n_layers, 6 * P.nh + 2 * P.nh * P.ds), np.float32) if taps else None
    lib().orc_m3_backbone_step(_p(out), _p(x), _p(P.flat), _p(ssm), _p(kst), _p(vst), _p(angle), _p(tp), c_int64(P.dm),
                               c_int64(P.ds), c_int64(P.expand), c_int64(P.hd), c_int64(P.ng), c_int64(P.n_layers),
                               c_int64(P.n_rope), c_float(P.a_floor), c_int(1 if P.outproj_norm else 0), c_int64(P.input_dim))
    if not taps:
        return out
    nh, ds = P.nh, P.ds
    res = []
    for l in range(P.n_layers):
        t = tp[l]
        res.append(dict(alpha=t[0:nh], beta=t[nh:2 * nh], gamma=t[2 * nh:3 * nh], dt=t[3 * nh:4 * nh], trap=t[4 * nh:5 * nh],
                        a_val=t[5 * nh:6 * nh], k=t[6 * nh:6 * nh + nh * ds].reshape(nh, ds),
                        q=t[6 * nh + nh * ds:].reshape(nh, ds)))
    return out, res


# ---- sampling (oracle/sample_oracle.c) -----------------------------------------------------------------

class Xoshiro:
    """Xoshiro256PlusPlus of src/module/sample.rs:48-86."""

    def __init__(self, seed=None, state=None):
        self.s = (c_uint64 * 4)()
        if state is not None:
            for i, v in enumerate(state):
                self.s[i] = v
        else:
            lib().orc_xoshiro_seed(c_uint64(seed), self.s)

    def state(self):
        return [int(v) for v in self.s]

    def next_u64(self):
        lib().orc_xoshiro_next_u64.restype = c_uint64
        return int(lib().orc_xoshiro_next_u64(self.s))

    def next_f32(self):
        lib().orc_xoshiro_next_f32.restype = c_float
        return float(lib().orc_xoshiro_next_f32(self.s))


def _filter(name, x, *args):
    x = np.array(x, dtype=np.float32, copy=True, order="C")
    getattr(lib(), name)(_p(x), c_int64(x.size), *args)
    return x


def apply_repetition_penalty(logits, seen, penalty):
    seen = np.ascontiguousarray(seen, dtype=np.uint32)
    return _filter("orc_apply_repetition_penalty", logits, _p(seen), c_int64(seen.size), c_float(penalty))


def apply_temperature(logits, t):
    return _filter("orc_apply_temperature", logits, c_float(t))


def apply_top_k(logits, k):
    return _filter("orc_apply_top_k", logits, c_int64(k))


def softmax(logits):
    return _filter("orc_softmax_inplace", logits)


def apply_top_p(probs, p):
    return _filter("orc_apply_top_p", probs, c_float(p))


def apply_min_p(probs, p):
    return _filter("orc_apply_min_p", probs, c_float(p))


def weighted_sample(probs, r):
    probs = _c(probs)
    lib().orc_weighted_sample.restype = ctypes.c_uint32
    return int(lib().orc_weighted_sample(_p(probs), c_int64(probs.size), c_float(r)))


def sample_token(logits, rng: Xoshiro, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, repetition_penalty=1.0, seen=()):
    """sample_token (src/module/sample.rs:243-265) -> (token, the logits buffer as the call leaves it)."""
    x = np.array(logits, dtype=np.float32, copy=True, order="C")
    seen = np.ascontiguousarray(seen, dtype=np.uint32)
    lib().orc_sample_token.restype = ctypes.c_uint32
    tok = lib().orc_sample_token(_p(x), c_int64(x.size), c_float(temperature), c_int64(top_k), c_float(top_p), c_float(min_p),
                                 c_float(repetition_penalty), _p(seen), c_int64(seen.size), rng.s)
    return int(tok), x
