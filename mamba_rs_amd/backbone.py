"""GpuMambaBackbone / GpuMambaLM: host mirror of the reference's engine types
(src/mamba_ssm/gpu/inference.rs:1515-1855, src/module/gpu_lm.rs:121-516) over the C ABI.

All arithmetic happens in libmamba_hip.so; this module only marshals numpy arrays.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from ctypes import c_uint64, POINTER, Structure, byref, c_float, c_int, c_void_p

import numpy as np

from . import _lib
from .config import MambaConfig, WeightDtype
from .weights import MambaWeights

_FP = POINTER(c_float)
_TOKEN_CB = ctypes.CFUNCTYPE(c_int, c_int, c_void_p)


class _CConfig(Structure):
    _fields_ = [("d_model", c_int), ("d_state", c_int), ("d_conv", c_int), ("expand", c_int), ("n_layers", c_int),
                ("scan_mode", c_int), ("rms_norm_eps", c_float)]


class _CLayer(Structure):
    _fields_ = [(n, _FP) for n in ("norm_weight", "in_proj_w", "conv1d_weight", "conv1d_bias", "x_proj_w", "dt_proj_w",
                                   "dt_proj_b", "a_log", "d_param", "out_proj_w")]


class _CWeights(Structure):
    _fields_ = [("input_proj_w", _FP), ("input_proj_b", _FP), ("layers", POINTER(_CLayer)), ("norm_f_weight", _FP)]


def _fp(a: np.ndarray):
    return a.ctypes.data_as(_FP)


def _bind():
    lib = _lib.load()
    if getattr(lib, "_engine_bound", False):
        return lib
    P = c_void_p
    sigs = {
        "mrs_backbone_create": (c_int, [POINTER(P), c_int, POINTER(_CWeights), POINTER(_CConfig), c_int, c_int, c_int]),
        "mrs_backbone_destroy": (None, [P]),
        "mrs_backbone_step": (c_int, [P, _FP, _FP]),
        "mrs_backbone_step_gpu_only": (c_int, [P]),
        "mrs_backbone_reset": (c_int, [P]),
        "mrs_backbone_capture_graph": (c_int, [P]),
        "mrs_backbone_alloc_prefill_scratch": (c_int, [P, c_int]),
        "mrs_backbone_prefill_sequence": (c_int, [P, _FP, c_int, _FP]),
        "mrs_backbone_prefill_device": (c_int, [P, P, c_int]),
        "mrs_backbone_temporal_ptr": (P, [P]),
        "mrs_backbone_temporal_dtype": (c_int, [P]),
        "mrs_backbone_decode_route": (c_int, [P]),
        "mrs_backbone_download_temporal": (c_int, [P, _FP]),
        "mrs_backbone_set_gemm_tuning": (c_int, [P, c_int]),
        "mrs_backbone_input_ptr": (P, [P]),
        "mrs_backbone_prefill_input_ptr": (P, [P]),
        "mrs_backbone_stream": (P, [P]),
        "mrs_backbone_sync": (c_int, [P]),
        "mrs_backbone_state_ptrs": (c_int, [P, c_int, POINTER(P), POINTER(P)]),
        "mrs_backbone_download_state": (c_int, [P, c_int, _FP, _FP]),
        "mrs_lm_create": (c_int, [POINTER(P), P, _FP, c_int]),
        "mrs_lm3_create": (c_int, [POINTER(P), P, _FP, c_int]),
        "mrs_lm_set_untied_head": (c_int, [P, _FP]),
        "mrs_lm_destroy": (None, [P]),
        "mrs_lm_set_tokens": (c_int, [P, POINTER(c_int)]),
        "mrs_lm_get_tokens": (c_int, [P, POINTER(c_int)]),
        "mrs_lm_decode_step": (c_int, [P]),
        "mrs_lm_capture_graph": (c_int, [P]),
        "mrs_lm_last_logits": (c_int, [P, _FP]),
        "mrs_lm_prefill": (c_int, [P, P, POINTER(c_int), c_int]),
        "mrs_lm_generate_batch": (c_int, [P, POINTER(c_int), POINTER(c_int), POINTER(_CSampleParams), c_int, POINTER(c_int), c_int,
                                          POINTER(c_int)]),
        "mrs_lm_generate_streaming": (c_int, [P, POINTER(c_int), c_int, POINTER(_CSampleParams), _TOKEN_CB, c_void_p]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    lib._engine_bound = True
    lib._engine_names = sorted(sigs)
    return lib


def engine_exported_names():
    return list(_bind()._engine_names)


class _CSampler(Structure):
    _fields_ = [("temperature", c_float), ("top_k", c_int), ("top_p", c_float), ("min_p", c_float), ("repetition_penalty", c_float)]


class _CSampleParams(Structure):
    _fields_ = [("sampler", _CSampler), ("max_tokens", c_int), ("eos_token_ids", POINTER(c_int)), ("n_eos", c_int), ("seed", c_uint64)]


@dataclass
class SampleParams:
    """SampleParams with the reference's defaults (src/module/sample.rs:20-46)."""
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    max_tokens: int = 256
    eos_token_ids: list = field(default_factory=list)
    seed: int = 42


def _call(name, *args):
    lib = _bind()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise _lib.MambaHipError(name, rc, lib.mrs_last_error().decode())


class GpuMambaBackbone:
    """One-GPU Mamba-1 backbone engine with fixed batch; `step` decodes one token per batch row,
    `prefill_sequence` runs whole sequences and leaves the state positioned for `step`."""

    def __init__(self, gpu_ordinal: int, weights: MambaWeights, cfg: MambaConfig, input_dim: int, batch: int,
                 dtype: WeightDtype = WeightDtype.F32):
        cfg.validate()
        weights.validate(cfg, input_dim)
        self.cfg, self.input_dim, self.batch, self.dtype = cfg, input_dim, batch, WeightDtype(dtype)
        keep = []

        def arr(a):
            a = np.ascontiguousarray(a, dtype=np.float32)
            keep.append(a)
            return _fp(a)

        layers = (_CLayer * cfg.n_layers)()
        for i, lw in enumerate(weights.layers):
            for n, _ in _CLayer._fields_:
                setattr(layers[i], n, arr(getattr(lw, n)))
        cw = _CWeights()
        identity = weights.input_proj_w.size == 0
        cw.input_proj_w = None if identity else arr(weights.input_proj_w)
        cw.input_proj_b = None if identity else arr(weights.input_proj_b)
        cw.layers = layers
        cw.norm_f_weight = arr(weights.norm_f_weight)
        cc = _CConfig(cfg.d_model, cfg.d_state, cfg.d_conv, cfg.expand, cfg.n_layers, int(cfg.scan_mode), cfg.rms_norm_eps)
        h = c_void_p()
        _call("mrs_backbone_create", byref(h), gpu_ordinal, byref(cw), byref(cc), input_dim, batch, int(self.dtype))
        self._h = h

    @classmethod
    def new(cls, gpu_ordinal, weights, cfg, input_dim, batch):
        return cls(gpu_ordinal, weights, cfg, input_dim, batch, WeightDtype.F32)

    @classmethod
    def new_with_dtype(cls, gpu_ordinal, weights, cfg, input_dim, batch, dtype):
        return cls(gpu_ordinal, weights, cfg, input_dim, batch, dtype)

    def close(self):
        if getattr(self, "_h", None):
            _bind().mrs_backbone_destroy(self._h)
            self._h = None

    __del__ = close

    def step(self, inp: np.ndarray) -> np.ndarray:
        inp = np.ascontiguousarray(inp, dtype=np.float32)
        if inp.size != self.batch * self.input_dim:
            raise ValueError(f"input must hold batch*input_dim = {self.batch * self.input_dim} values")
        out = np.empty((self.batch, self.cfg.d_model), np.float32)
        _call("mrs_backbone_step", self._h, _fp(inp), _fp(out))
        return out

    def step_gpu_only(self):
        _call("mrs_backbone_step_gpu_only", self._h)

    def reset(self):
        _call("mrs_backbone_reset", self._h)

    def capture_graph(self):
        _call("mrs_backbone_capture_graph", self._h)

    def alloc_prefill_scratch(self, T: int):
        _call("mrs_backbone_alloc_prefill_scratch", self._h, T)

    def prefill_sequence(self, inp: np.ndarray) -> np.ndarray:
        """inp [batch, T, input_dim] f32 -> norm_f output of the last position [batch, d_model]."""
        inp = np.ascontiguousarray(inp, dtype=np.float32)
        if inp.ndim != 3 or inp.shape[0] != self.batch or inp.shape[2] != self.input_dim:
            raise ValueError("input must be [batch, T, input_dim]")
        out = np.empty((self.batch, self.cfg.d_model), np.float32)
        _call("mrs_backbone_prefill_sequence", self._h, _fp(inp), inp.shape[1], _fp(out))
        return out

    prefill_sequence_mixed = prefill_sequence

    def prefill_device(self, ptr: int, T: int):
        _call("mrs_backbone_prefill_device", self._h, c_void_p(ptr), T)

    def sync(self):
        _call("mrs_backbone_sync", self._h)

    def set_gemm_tuning(self, on: bool = True):
        """Time the GEMM library's kernels for each projection shape once and keep the fastest (a few seconds per shape
        at the first prefill of a given length, or at the eager decode step that precedes capture_graph when the batch
        is past the own chain's row limit: call it before capturing)."""
        _call("mrs_backbone_set_gemm_tuning", self._h, 1 if on else 0)

    def temporal_ptr(self) -> int:
        return _bind().mrs_backbone_temporal_ptr(self._h)

    def download_temporal(self) -> np.ndarray:
        """download_temporal (inference.rs:1727-1737): final-norm rows of the last step / prefill, [batch, d_model]."""
        out = np.empty((self.batch, self.cfg.d_model), np.float32)
        _call("mrs_backbone_download_temporal", self._h, _fp(out))
        return out

    def temporal_dtype(self) -> WeightDtype:
        return WeightDtype(_bind().mrs_backbone_temporal_dtype(self._h))

    def decode_route(self) -> int:
        """0: chain on the vendor GEMM, 1: the library's own fused chain, 2: a whole step in one launch."""
        return _bind().mrs_backbone_decode_route(self._h)

    def input_ptr(self) -> int:
        return _bind().mrs_backbone_input_ptr(self._h)

    def prefill_input_ptr(self) -> int:
        return _bind().mrs_backbone_prefill_input_ptr(self._h)

    def stream(self) -> int:
        return _bind().mrs_backbone_stream(self._h)

    def download_state(self, layer: int):
        """(conv_state [batch, d_inner, d_conv], ssm_state [batch, d_inner, d_state]) of one layer."""
        di = self.cfg.d_inner()
        conv = np.empty((self.batch, di, self.cfg.d_conv), np.float32)
        ssm = np.empty((self.batch, di, self.cfg.d_state), np.float32)
        _call("mrs_backbone_download_state", self._h, layer, _fp(conv), _fp(ssm))
        return conv, ssm


class GpuMambaLM:
    """LM loop on top of a backbone (identity input_proj): GpuMambaLM (src/module/gpu_lm.rs:121-516) over a
    GpuMambaBackbone, GpuMamba3LM (src/module/gpu_lm3.rs:54-400) over a GpuMamba3Backbone.  The head is the embedding
    table (tied) unless `lm_head` [d_model, vocab] is given (GpuMambaLM::new, gpu_lm.rs:143-262)."""

    def __init__(self, backbone, embed: np.ndarray, lm_head: np.ndarray | None = None):
        self.backbone = backbone
        embed = np.ascontiguousarray(embed, dtype=np.float32)
        if embed.ndim != 2 or embed.shape[1] != backbone.cfg.d_model:
            raise ValueError("embed must be [vocab, d_model]")
        self.vocab = embed.shape[0]
        h = c_void_p()
        self._m1 = isinstance(backbone, GpuMambaBackbone)
        _call("mrs_lm_create" if self._m1 else "mrs_lm3_create", byref(h), backbone._h, _fp(embed), self.vocab)
        self._h = h
        if lm_head is not None:
            lm_head = np.ascontiguousarray(lm_head, dtype=np.float32)
            if lm_head.shape != (backbone.cfg.d_model, self.vocab):
                raise ValueError("lm_head must be [d_model, vocab]")
            _call("mrs_lm_set_untied_head", self._h, _fp(lm_head))

    @classmethod
    def from_hf(cls, directory: str, batch: int = 1, dtype: WeightDtype = WeightDtype.F32, gpu_ordinal: int = 0) -> "GpuMambaLM":
        """Engine + LM loop from a HuggingFace Mamba-1 checkpoint directory (hf::load_hf then GpuMambaLM::new,
        src/hf/load.rs:40, src/module/gpu_lm.rs:143)."""
        from .formats import load_hf
        m = load_hf(directory)
        bb = GpuMambaBackbone(gpu_ordinal, m.weights, m.cfg, m.cfg.d_model, batch, dtype)
        lm = cls(bb, m.embed[:m.vocab_size], m.lm_head)
        lm.hf = m.hf
        return lm

    def close(self):
        if getattr(self, "_h", None):
            _bind().mrs_lm_destroy(self._h)
            self._h = None

    __del__ = close

    def set_tokens(self, tokens):
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        _call("mrs_lm_set_tokens", self._h, t.ctypes.data_as(POINTER(c_int)))

    def get_tokens(self) -> np.ndarray:
        t = np.empty(self.backbone.batch, np.int32)
        _call("mrs_lm_get_tokens", self._h, t.ctypes.data_as(POINTER(c_int)))
        return t

    def decode_step(self):
        _call("mrs_lm_decode_step", self._h)

    def capture_graph(self):
        _call("mrs_lm_capture_graph", self._h)

    def last_logits(self) -> np.ndarray:
        out = np.empty((self.backbone.batch, self.vocab), np.float32)
        _call("mrs_lm_last_logits", self._h, _fp(out))
        return out

    def prefill(self, tokens: np.ndarray, engine: GpuMambaBackbone | None = None):
        """tokens [batch, T] through the backbone's prefill; `engine`: another Mamba-1 engine to run it on (its batch)."""
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        if t.ndim != 2 or t.shape[0] != (engine or self.backbone).batch:
            raise ValueError("tokens must be [batch, T]")
        _call("mrs_lm_prefill", self._h, engine._h if engine is not None else None, t.ctypes.data_as(POINTER(c_int)), t.shape[1])

    def generate_batch(self, prompts, params, *, seen_includes_prompt: bool = False):
        """GpuMambaLM::generate_batch (src/module/gpu_lm.rs:389-516): one prompt (any length) and one SampleParams per
        batch slot -> one list of generated tokens per slot.  The loop runs on the device."""
        B = self.backbone.batch
        if len(prompts) != B or len(params) != B:
            raise ValueError("prompts and params must have one entry per batch slot")
        lens = np.asarray([len(p) for p in prompts], np.int32)
        flat = np.ascontiguousarray(np.concatenate([np.asarray(p, np.int32).ravel() for p in prompts] + [np.zeros(0, np.int32)]))
        cp = (_CSampleParams * B)()
        keep = []
        for i, sp in enumerate(params):
            eos = np.ascontiguousarray(sp.eos_token_ids, dtype=np.int32)
            keep.append(eos)
            cp[i].sampler = _CSampler(sp.temperature, sp.top_k, sp.top_p, sp.min_p, sp.repetition_penalty)
            cp[i].max_tokens, cp[i].n_eos, cp[i].seed = sp.max_tokens, eos.size, sp.seed & 0xFFFFFFFFFFFFFFFF
            cp[i].eos_token_ids = eos.ctypes.data_as(POINTER(c_int)) if eos.size else None
        stride = max(1, max(sp.max_tokens for sp in params))
        out = np.zeros((B, stride), np.int32)
        out_lens = np.zeros(B, np.int32)
        _call("mrs_lm_generate_batch", self._h, flat.ctypes.data_as(POINTER(c_int)), lens.ctypes.data_as(POINTER(c_int)), cp,
              1 if seen_includes_prompt else 0, out.ctypes.data_as(POINTER(c_int)), stride, out_lens.ctypes.data_as(POINTER(c_int)))
        return [[int(t) for t in out[i, :out_lens[i]]] for i in range(B)]

    def generate_streaming(self, prompt, params: SampleParams, callback):
        """GpuMambaLM::generate_streaming (gpu_lm.rs:334-377), batch-1 engines: `callback(token)` runs for every new
        token as soon as it exists; a true return value ends the generation early.  Returns nothing."""
        if self.backbone.batch != 1:
            raise ValueError("generate_streaming requires batch=1; use generate_batch for batch>1")
        p = np.ascontiguousarray(list(prompt), dtype=np.int32)
        eos = np.ascontiguousarray(params.eos_token_ids, dtype=np.int32)
        cp = _CSampleParams()
        cp.sampler = _CSampler(params.temperature, params.top_k, params.top_p, params.min_p, params.repetition_penalty)
        cp.max_tokens, cp.n_eos, cp.seed = params.max_tokens, eos.size, params.seed & 0xFFFFFFFFFFFFFFFF
        cp.eos_token_ids = eos.ctypes.data_as(POINTER(c_int)) if eos.size else None
        raised = []

        def trampoline(token, _user):
            try:
                return 1 if callback(int(token)) else 0
            except BaseException as e:   # an exception must not unwind through the C frames: stop, re-raise after the call
                raised.append(e)
                return 1

        _call("mrs_lm_generate_streaming", self._h, p.ctypes.data_as(POINTER(c_int)) if p.size else None, int(p.size), byref(cp),
              _TOKEN_CB(trampoline), None)
        if raised:
            raise raised[0]

    def generate(self, prompt, max_tokens: int | None = None, params: SampleParams | None = None):
        """GpuMambaLM::generate for a batch-1 engine (gpu_lm.rs:323-377).  With `params` the reference's sampled loop
        (penalty over prompt + generated tokens, EOS, seed); with `max_tokens` alone the greedy loop, where the prompt
        goes through prefill when it has at least 2 tokens, token by token otherwise."""
        if self.backbone.batch != 1:
            raise ValueError("generate() is the batch-1 entry point")
        if params is not None:
            return self.generate_batch([list(prompt)], [params], seen_includes_prompt=True)[0]
        prompt = list(prompt)
        self.backbone.reset()
        if len(prompt) >= 2:
            self.prefill(np.asarray([prompt], np.int32))
        else:
            self.set_tokens(prompt[:1])
            self.decode_step()
        out = [int(self.get_tokens()[0])]
        for _ in range(max_tokens - 1):
            self.decode_step()
            out.append(int(self.get_tokens()[0]))
        return out
