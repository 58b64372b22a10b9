"""On-disk formats either side of the hot path (host side only; no GPU work here).

* Native checkpoints: the reference's safetensors layout (src/serialize.rs:31-252) -- tensor names
  `input_proj.*`, `layers.{i}.*`, `norm_f.weight`, all f32, row-major `[n_in, n_out]`, and a `config` metadata
  string -- so files written here load in the reference and the other way round.
* Native Mamba-3 SISO checkpoints: src/mamba3_siso/serialize.rs:28-150 (its own tensor names and one metadata
  entry per config field).
* HuggingFace Mamba-1 checkpoints (`state-spaces/mamba-*-hf` and the original `mamba_ssm` naming): config.json
  parsing (src/hf/config_json.rs), tensor-key remapping (src/hf/keys.rs), the `[out, in] -> [in, out]` transposes,
  embedding padding to a multiple of 64 rows and the tied / untied head (src/hf/load.rs:40-326).
"""
from __future__ import annotations

import json
import os
import re
from dataclasses import dataclass

import numpy as np

from .config import MambaConfig, ScanMode
from .weights import MambaLayerWeights, MambaWeights

# ---- native format (src/serialize.rs) ------------------------------------------------------------------

_LAYER_TENSORS = (  # (file suffix, MambaLayerWeights field, shape as a function of the dims)
    ("norm.weight", "norm_weight", lambda d: (d["dm"],)),
    ("in_proj.weight", "in_proj_w", lambda d: (d["dm"], 2 * d["di"])),
    ("conv1d.weight", "conv1d_weight", lambda d: (d["di"], d["dc"])),
    ("conv1d.bias", "conv1d_bias", lambda d: (d["di"],)),
    ("x_proj.weight", "x_proj_w", lambda d: (d["di"], d["xd"])),
    ("dt_proj.weight", "dt_proj_w", lambda d: (d["dr"], d["di"])),
    ("dt_proj.bias", "dt_proj_b", lambda d: (d["di"],)),
    ("a_log", "a_log", lambda d: (d["di"], d["ds"])),
    ("D", "d_param", lambda d: (d["di"],)),
    ("out_proj.weight", "out_proj_w", lambda d: (d["di"], d["dm"])),
)
_SCAN_MODE_NAMES = {ScanMode.SEQUENTIAL: "Sequential", ScanMode.PARALLEL: "Parallel", ScanMode.AUTO: "Auto"}


def _dims(cfg: MambaConfig) -> dict:
    return dict(dm=cfg.d_model, di=cfg.d_inner(), ds=cfg.d_state, dc=cfg.d_conv, dr=cfg.dt_rank(), xd=cfg.xdbl_dim())


def _f32_plain(v: float) -> str:
    """An f32 the way Rust's `{}` prints it: shortest round-trip digits, positional (1e-5 -> 0.00001)."""
    return np.format_float_positional(np.float32(v), trim="-")


def save(path: str, weights: MambaWeights, cfg: MambaConfig, input_dim: int) -> None:
    """serialize::save (src/serialize.rs:31-113)."""
    from safetensors.numpy import save_file
    cfg.validate()
    weights.validate(cfg, input_dim)
    d = _dims(cfg)
    f = lambda a, shape: np.ascontiguousarray(np.asarray(a, dtype=np.float32).reshape(shape))
    tensors = {"input_proj.weight": f(weights.input_proj_w, (input_dim, d["dm"]) if weights.input_proj_w.size else (0, d["dm"])),
               "input_proj.bias": f(weights.input_proj_b, (-1,))}
    for i, lw in enumerate(weights.layers):
        for suffix, field, shape in _LAYER_TENSORS:
            tensors[f"layers.{i}.{suffix}"] = f(getattr(lw, field), shape(d))
    tensors["norm_f.weight"] = f(weights.norm_f_weight, (d["dm"],))
    meta = ('{"d_model":%d,"d_state":%d,"d_conv":%d,"expand":%d,"n_layers":%d,"input_dim":%d,"scan_mode":"%s","rms_norm_eps":%s}'
            % (cfg.d_model, cfg.d_state, cfg.d_conv, cfg.expand, cfg.n_layers, input_dim, _SCAN_MODE_NAMES[ScanMode(cfg.scan_mode)],
               _f32_plain(cfg.rms_norm_eps)))
    save_file(tensors, path, metadata={"config": meta})


def _parse_usize(meta: str, key: str) -> int:
    m = re.search(r'"%s":(\d+)' % re.escape(key), meta)
    if not m:
        raise ValueError(f"missing '{key}' in config metadata")
    return int(m.group(1))


def load(path: str):
    """serialize::load (src/serialize.rs:115-252) -> (weights, cfg, input_dim).  Tensors must be f32."""
    from safetensors import safe_open
    with safe_open(path, framework="np") as st:
        meta = (st.metadata() or {}).get("config")
        if meta is None:
            raise ValueError("missing 'config' metadata")
        dm, ds, dc = _parse_usize(meta, "d_model"), _parse_usize(meta, "d_state"), _parse_usize(meta, "d_conv")
        expand, n_layers, input_dim = _parse_usize(meta, "expand"), _parse_usize(meta, "n_layers"), _parse_usize(meta, "input_dim")
        scan_mode = ScanMode.SEQUENTIAL if '"scan_mode":"Sequential"' in meta else ScanMode.PARALLEL if '"scan_mode":"Parallel"' in meta else ScanMode.AUTO
        m = re.search(r'"rms_norm_eps":([0-9.e-]+)', meta)
        eps = float(m.group(1)) if m else MambaConfig().rms_norm_eps
        cfg = MambaConfig(d_model=dm, d_state=ds, d_conv=dc, expand=expand, n_layers=n_layers, scan_mode=scan_mode, rms_norm_eps=eps)
        cfg.validate()
        names = set(st.keys())

        def read(name):
            if name not in names:
                raise ValueError(f"tensor '{name}': not found")
            a = st.get_tensor(name)
            if a.dtype != np.float32:
                raise ValueError(f"tensor '{name}': dtype {a.dtype}, expected F32")
            return np.ascontiguousarray(a)

        layers = []
        for i in range(n_layers):
            layers.append(MambaLayerWeights(**{field: read(f"layers.{i}.{suffix}") for suffix, field, _ in _LAYER_TENSORS}))
        w = MambaWeights(read("input_proj.weight"), read("input_proj.bias"), layers, read("norm_f.weight"))
    w.validate(cfg, input_dim)
    return w, cfg, input_dim


# ---- native Mamba-3 SISO format (src/mamba3_siso/serialize.rs) ------------------------------------------

_M3_LAYER_TENSORS = (
    ("norm.weight", "norm_weight", lambda c: (c.d_model,)),
    ("in_proj.weight", "in_proj_w", lambda c: (c.d_model, c.in_proj_out_dim())),
    ("dt_bias", "dt_bias", lambda c: (c.nheads(),)),
    ("b_norm.weight", "b_norm_weight", lambda c: (c.d_state,)),
    ("c_norm.weight", "c_norm_weight", lambda c: (c.d_state,)),
    ("b_bias", "b_bias", lambda c: (c.nheads(), c.d_state)),
    ("c_bias", "c_bias", lambda c: (c.nheads(), c.d_state)),
    ("D", "d_param", lambda c: (c.nheads(),)),
    ("norm_gate.weight", "norm_gate_weight", lambda c: (c.d_inner(),)),
    ("out_proj.weight", "out_proj_w", lambda c: (c.d_inner(), c.d_model)),
)


def save_mamba3(path: str, weights, cfg, input_dim: int) -> None:
    """save_mamba3 (src/mamba3_siso/serialize.rs:28-91)."""
    from safetensors.numpy import save_file
    weights.validate(cfg, input_dim)
    f = lambda a, shape: np.ascontiguousarray(np.asarray(a, dtype=np.float32).reshape(shape))
    tensors = {"input_proj.weight": f(weights.input_proj_w, (input_dim if weights.input_proj_w.size else 0, cfg.d_model)),
               "input_proj.bias": f(weights.input_proj_b, (-1,))}
    for i, lw in enumerate(weights.layers):
        for suffix, field, shape in _M3_LAYER_TENSORS:
            tensors[f"layers.{i}.{suffix}"] = f(getattr(lw, field), shape(cfg))
    tensors["norm_f.weight"] = f(weights.norm_f_weight, (cfg.d_model,))
    meta = {"d_model": str(cfg.d_model), "d_state": str(cfg.d_state), "expand": str(cfg.expand), "headdim": str(cfg.headdim),
            "ngroups": str(cfg.ngroups), "n_layers": str(cfg.n_layers), "input_dim": str(input_dim),
            "rope_fraction": _f32_plain(cfg.rope_fraction), "a_floor": _f32_plain(cfg.a_floor), "mamba_version": "3"}
    save_file(tensors, path, metadata=meta)


def load_mamba3(path: str, cfg):
    """load_mamba3 (src/mamba3_siso/serialize.rs:93-150) -> (weights, input_dim); the caller brings the config, the
    file brings input_dim and f32 tensors."""
    from safetensors import safe_open
    from .mamba3 import Mamba3LayerWeights, Mamba3Weights
    with safe_open(path, framework="np") as st:
        meta = st.metadata()
        if meta is None:
            raise ValueError("no metadata")
        if "input_dim" not in meta:
            raise ValueError("missing input_dim")
        try:
            input_dim = int(meta["input_dim"])
        except ValueError as e:
            raise ValueError(f"parse input_dim: {e}")
        names = set(st.keys())

        def read(name):
            if name not in names:
                raise ValueError(f"tensor '{name}': not found")
            a = st.get_tensor(name)
            if a.dtype != np.float32:
                raise ValueError(f"tensor '{name}': dtype {a.dtype}, expected F32")
            return np.ascontiguousarray(a)

        layers = [Mamba3LayerWeights(**{field: read(f"layers.{i}.{suffix}") for suffix, field, _ in _M3_LAYER_TENSORS})
                  for i in range(cfg.n_layers)]
        w = Mamba3Weights(read("input_proj.weight"), read("input_proj.bias"), layers, read("norm_f.weight"))
    w.validate(cfg, input_dim)
    return w, input_dim


# ---- HuggingFace config.json (src/hf/config_json.rs) ---------------------------------------------------

@dataclass
class HfMambaConfig:
    family: str              # "mamba1" | "mamba2"
    d_model: int
    n_layers: int
    d_state: int
    d_conv: int
    expand: int
    vocab_size: int
    tie_word_embeddings: bool
    use_bias: bool
    use_conv_bias: bool
    rms_norm_eps: float


def parse_config_json(data) -> HfMambaConfig:
    """parse_config_json (config_json.rs:64-132): HF-native (`hidden_size`, ...) or original (`d_model`, `n_layer`) fields."""
    try:
        raw = data if isinstance(data, dict) else json.loads(data)
    except (ValueError, TypeError) as e:
        raise ValueError(f"config.json parse error: {e}")
    mt = raw.get("model_type")
    if mt is not None:
        if mt in ("mamba", "falcon_mamba"):
            family = "mamba1"
        elif mt == "mamba2":
            family = "mamba2"
        else:
            raise ValueError(f"unsupported model_type: {mt}")
    elif raw.get("d_model") is not None:
        family = "mamba1"
    else:
        raise ValueError("cannot detect model family: no model_type or d_model field")

    def need(key, what):
        v = raw.get(key)
        if v is None:
            raise ValueError(f"{what} missing {key}")
        return int(v)

    if mt is not None or raw.get("hidden_size") is not None:
        d_model, n_layers = need("hidden_size", "HF config"), need("num_hidden_layers", "HF config")
        d_state, d_conv = need("state_size", "HF config"), need("conv_kernel", "HF config")
    else:
        d_model, n_layers = need("d_model", "original config"), need("n_layer", "original config")
        d_state, d_conv = int(raw.get("d_state") or 16), int(raw.get("d_conv") or 4)
    if raw.get("vocab_size") is None:
        raise ValueError("missing vocab_size in config.json")
    tsr = raw.get("time_step_rank")
    if tsr is not None and int(tsr) != -(-d_model // 16):
        raise ValueError(f"time_step_rank mismatch: config has {tsr}, expected d_model.div_ceil(16) = {-(-d_model // 16)}")
    eps = raw.get("rms_norm_eps")
    if eps is None:
        eps = raw.get("layer_norm_epsilon")
    tie = raw.get("tie_word_embeddings")
    ub, ucb = raw.get("use_bias"), raw.get("use_conv_bias")
    return HfMambaConfig(family, d_model, n_layers, d_state, d_conv, int(raw.get("expand") or 2), int(raw["vocab_size"]),
                         True if tie is None else bool(tie), False if ub is None else bool(ub), True if ucb is None else bool(ucb),
                         1e-5 if eps is None else float(eps))


# ---- HuggingFace tensor keys (src/hf/keys.rs) ----------------------------------------------------------

_HF_LAYER_FIELDS = {
    "mixer.in_proj.weight": "in_proj_w", "mixer.conv1d.weight": "conv1d_weight", "mixer.conv1d.bias": "conv1d_bias",
    "mixer.x_proj.weight": "x_proj_w", "mixer.dt_proj.weight": "dt_proj_w", "mixer.dt_proj.bias": "dt_proj_b",
    "mixer.A_log": "a_log", "mixer.D": "d_param", "mixer.out_proj.weight": "out_proj_w", "norm.weight": "norm_weight",
}


def remap_m1_hf_key(key: str):
    """remap_m1_hf_key (keys.rs:19-58): ("layer", index, field) | ("norm_f",) | ("embedding",) | ("lm_head",) | ("unknown",)."""
    if key in ("backbone.embeddings.weight", "backbone.embedding.weight"):
        return ("embedding",)
    if key == "lm_head.weight":
        return ("lm_head",)
    if key == "backbone.norm_f.weight":
        return ("norm_f",)
    if key.startswith("backbone.layers."):
        rest = key[len("backbone.layers."):]
        if "." not in rest:
            return ("unknown",)
        idx, suffix = rest.split(".", 1)
        if not (idx.isascii() and idx.isdigit()):
            return ("unknown",)
        field = _HF_LAYER_FIELDS.get(suffix)
        return ("layer", int(idx), field) if field else ("unknown",)
    return ("unknown",)


# ---- HuggingFace checkpoint directory (src/hf/load.rs) -------------------------------------------------

@dataclass
class HfModel:
    cfg: MambaConfig
    weights: MambaWeights         # identity input projection (empty input_proj_w)
    embed: np.ndarray             # [vocab_size_padded, d_model] f32, rows past vocab_size zero
    lm_head: np.ndarray | None    # [d_model, vocab_size] f32 when the head is not tied, else None
    vocab_size: int
    vocab_size_padded: int
    hf: HfMambaConfig


def _discover_shards(directory: str):
    index = os.path.join(directory, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index) as fh:
            wm = json.load(fh).get("weight_map")
        if not isinstance(wm, dict):
            raise ValueError("index.json missing weight_map")
        return [os.path.join(directory, f) for f in sorted(set(v for v in wm.values() if isinstance(v, str)))]
    single = os.path.join(directory, "model.safetensors")
    if os.path.exists(single):
        return [single]
    raise ValueError(f"no model.safetensors or index.json in {directory}")


def _tensor_f32(st, name) -> np.ndarray:
    """f32 / bf16 / f16 tensors widened to f32 (tensor_to_f32, load.rs:231-250); anything else is refused."""
    import torch
    t = st.get_tensor(name)
    if t.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise ValueError(f"unsupported dtype: {t.dtype}")
    return t.to(torch.float32).contiguous().numpy()


def load_hf(directory: str) -> HfModel:
    """load_hf (load.rs:40-214): config.json + model.safetensors (or shards named by model.safetensors.index.json)."""
    from safetensors import safe_open
    with open(os.path.join(directory, "config.json"), "rb") as fh:
        hf = parse_config_json(fh.read())
    if hf.family != "mamba1":
        raise ValueError("load_hf reads Mamba-1 checkpoints")
    if not 0 < hf.vocab_size <= 1 << 24:
        raise ValueError(f"vocab_size {hf.vocab_size} out of supported range (1..=2^24)")
    if not 0 < hf.d_model <= 1 << 20:
        raise ValueError(f"d_model {hf.d_model} out of supported range (1..=2^20)")
    if hf.use_bias:
        raise ValueError("HF config has use_bias=true (non-default): projection biases are not part of the inference kernels")
    cfg = MambaConfig(d_model=hf.d_model, d_state=hf.d_state, d_conv=hf.d_conv, expand=hf.expand, n_layers=hf.n_layers,
                      rms_norm_eps=hf.rms_norm_eps)
    cfg.validate()
    dm, di, ds, dc, dr, xd = cfg.d_model, cfg.d_inner(), cfg.d_state, cfg.d_conv, cfg.dt_rank(), cfg.xdbl_dim()
    vpad = (hf.vocab_size + 63) & ~63
    embed = np.zeros((vpad, dm), np.float32)
    lm_head = None
    norm_f = None
    fields = [dict() for _ in range(hf.n_layers)]
    for shard in _discover_shards(directory):
        with safe_open(shard, framework="pt") as st:
            for name in st.keys():
                kind = remap_m1_hf_key(name)
                if kind[0] == "unknown":
                    continue
                data = _tensor_f32(st, name)
                if kind[0] == "embedding":
                    if data.size != hf.vocab_size * dm:
                        raise ValueError(f"embedding shape: expected {hf.vocab_size * dm} elements, got {data.size}")
                    embed[:hf.vocab_size] = data.reshape(hf.vocab_size, dm)
                elif kind[0] == "lm_head":
                    lm_head = data
                elif kind[0] == "norm_f":
                    if data.size != dm:
                        raise ValueError(f"norm_f_weight: expected {dm}, got {data.size}")
                    norm_f = data.reshape(dm)
                else:
                    _, idx, field = kind
                    if idx >= hf.n_layers:
                        raise ValueError(f"layer index {idx} >= n_layers {hf.n_layers}")
                    if field in fields[idx]:
                        raise ValueError(f"duplicate field: {field}")
                    fields[idx][field] = data
    if not hf.tie_word_embeddings and lm_head is None:
        raise ValueError("tie_word_embeddings=false but lm_head.weight not found")
    if hf.tie_word_embeddings:
        lm_head = None
    if lm_head is not None:
        if lm_head.size != hf.vocab_size * dm:
            raise ValueError(f"lm_head.weight: expected {hf.vocab_size * dm} elements, got {lm_head.size}")
        lm_head = np.ascontiguousarray(lm_head.reshape(hf.vocab_size, dm).T)
    if norm_f is None:
        norm_f = np.zeros(dm, np.float32)   # the reference starts from zeros and copies what the file holds

    def take(i, field, n):
        if field not in fields[i]:
            raise ValueError(f"layer {i}: missing field: {field}")
        a = fields[i].pop(field)
        if a.size != n:
            raise ValueError(f"layer {i}: {field} has {a.size} elements, expected {n}")
        return a

    layers = []
    for i in range(hf.n_layers):
        if not fields[i]:
            raise ValueError(f"layer {i}: no weights found")
        tr = lambda a, rows, cols: np.ascontiguousarray(a.reshape(rows, cols).T)   # PyTorch [out, in] -> [in, out]
        layers.append(MambaLayerWeights(
            norm_weight=take(i, "norm_weight", dm).reshape(dm),
            in_proj_w=tr(take(i, "in_proj_w", 2 * di * dm), 2 * di, dm),
            conv1d_weight=take(i, "conv1d_weight", di * dc).reshape(di, dc),   # [d_inner, 1, d_conv] squeezed: no transpose
            conv1d_bias=take(i, "conv1d_bias", di).reshape(di) if hf.use_conv_bias else np.zeros(di, np.float32),
            x_proj_w=tr(take(i, "x_proj_w", xd * di), xd, di),
            dt_proj_w=tr(take(i, "dt_proj_w", di * dr), di, dr),
            dt_proj_b=take(i, "dt_proj_b", di).reshape(di),
            a_log=take(i, "a_log", di * ds).reshape(di, ds),
            d_param=take(i, "d_param", di).reshape(di),
            out_proj_w=tr(take(i, "out_proj_w", dm * di), dm, di)))
    weights = MambaWeights(np.zeros((0, dm), np.float32), np.zeros(0, np.float32), layers, norm_f)
    return HfModel(cfg, weights, embed, lm_head, hf.vocab_size, vpad, hf)


def save_hf(directory: str, cfg: MambaConfig, weights: MambaWeights, embed: np.ndarray, vocab_size: int, *, dtype: str = "float32",
            lm_head: np.ndarray | None = None, shards: int = 1) -> None:
    """Writes an HF-native Mamba-1 checkpoint directory (config.json + model.safetensors, or `shards` files plus
    model.safetensors.index.json) with PyTorch layouts: nn.Linear weights `[out, in]`, conv1d `[d_inner, 1, d_conv]`.
    The inverse of load_hf; the reference only reads this format."""
    import torch
    from safetensors.torch import save_file
    os.makedirs(directory, exist_ok=True)
    tdt = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}[dtype]
    dm, di, dc = cfg.d_model, cfg.d_inner(), cfg.d_conv
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(tdt).contiguous()
    tensors = {"backbone.embeddings.weight": t(np.asarray(embed, np.float32)[:vocab_size]), "backbone.norm_f.weight": t(weights.norm_f_weight)}
    for i, lw in enumerate(weights.layers):
        p = f"backbone.layers.{i}."
        tensors[p + "norm.weight"] = t(lw.norm_weight)
        tensors[p + "mixer.in_proj.weight"] = t(np.asarray(lw.in_proj_w).reshape(dm, 2 * di).T)
        tensors[p + "mixer.conv1d.weight"] = t(np.asarray(lw.conv1d_weight).reshape(di, 1, dc))
        tensors[p + "mixer.conv1d.bias"] = t(lw.conv1d_bias)
        tensors[p + "mixer.x_proj.weight"] = t(np.asarray(lw.x_proj_w).reshape(di, cfg.xdbl_dim()).T)
        tensors[p + "mixer.dt_proj.weight"] = t(np.asarray(lw.dt_proj_w).reshape(cfg.dt_rank(), di).T)
        tensors[p + "mixer.dt_proj.bias"] = t(lw.dt_proj_b)
        tensors[p + "mixer.A_log"] = t(lw.a_log)
        tensors[p + "mixer.D"] = t(lw.d_param)
        tensors[p + "mixer.out_proj.weight"] = t(np.asarray(lw.out_proj_w).reshape(di, dm).T)
    if lm_head is not None:
        tensors["lm_head.weight"] = t(np.asarray(lm_head, np.float32).reshape(dm, vocab_size).T)
    with open(os.path.join(directory, "config.json"), "w") as fh:
        json.dump({"model_type": "mamba", "hidden_size": dm, "num_hidden_layers": cfg.n_layers, "state_size": cfg.d_state,
                   "conv_kernel": dc, "expand": cfg.expand, "vocab_size": vocab_size, "time_step_rank": cfg.dt_rank(),
                   "tie_word_embeddings": lm_head is None, "use_bias": False, "use_conv_bias": True,
                   "rms_norm_eps": float(cfg.rms_norm_eps)}, fh)
    names = sorted(tensors)
    if shards <= 1:
        save_file(tensors, os.path.join(directory, "model.safetensors"))
        return
    weight_map = {}
    for s in range(shards):
        part = {n: tensors[n] for n in names[s::shards]}
        fname = f"model-{s + 1:05d}-of-{shards:05d}.safetensors"
        save_file(part, os.path.join(directory, fname))
        weight_map.update({n: fname for n in part})
    with open(os.path.join(directory, "model.safetensors.index.json"), "w") as fh:
        json.dump({"metadata": {}, "weight_map": weight_map}, fh)
