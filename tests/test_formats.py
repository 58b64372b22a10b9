"""On-disk formats: the native safetensors layout (src/serialize.rs) and HuggingFace Mamba-1 checkpoints (src/hf/).

Test vectors are the reference's own: the key-remap cases of src/hf/keys.rs:60-136, the config.json cases of
src/hf/config_json.rs:134-232, the round trip of tests/m1_test_correctness.rs:152-195 and the synthetic checkpoint
of tests/hf_integration.rs:15-176 (same shapes, same xorshift fill, written here with plain safetensors so the
loader is checked against a writer that shares no code with it).
"""
import json
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from mamba_rs_amd import MambaConfig, MambaWeights, ScanMode  # noqa: E402
from mamba_rs_amd import formats  # noqa: E402
from mamba_rs_amd.formats import load_hf, parse_config_json, remap_m1_hf_key, save_hf  # noqa: E402


# ---- keys.rs --------------------------------------------------------------------------------------------

@pytest.mark.parametrize("key,want", [
    ("backbone.layers.3.mixer.in_proj.weight", ("layer", 3, "in_proj_w")),
    ("backbone.layers.0.mixer.A_log", ("layer", 0, "a_log")),
    ("backbone.layers.5.mixer.D", ("layer", 5, "d_param")),
    ("backbone.layers.0.mixer.conv1d.weight", ("layer", 0, "conv1d_weight")),
    ("backbone.layers.12.norm.weight", ("layer", 12, "norm_weight")),
    ("backbone.embeddings.weight", ("embedding",)),
    ("backbone.embedding.weight", ("embedding",)),
    ("lm_head.weight", ("lm_head",)),
    ("backbone.norm_f.weight", ("norm_f",)),
    ("something.else.weight", ("unknown",)),
    ("backbone.layers.0", ("unknown",)),
    ("backbone.layers.", ("unknown",)),
    ("backbone.layers.x.mixer.D", ("unknown",)),
    ("backbone.layers.0.mixer.in_proj.bias", ("unknown",)),
])
def test_remap_m1_hf_key(key, want):
    assert remap_m1_hf_key(key) == want


# ---- config_json.rs -------------------------------------------------------------------------------------

_MIN_HF = '{"model_type":"%s","hidden_size":64,"num_hidden_layers":2,"state_size":8,"conv_kernel":4,"vocab_size":100}'


def test_parse_hf_native_config():
    c = parse_config_json(b'{"model_type": "mamba", "hidden_size": 768, "num_hidden_layers": 24, "state_size": 16,'
                          b' "conv_kernel": 4, "expand": 2, "vocab_size": 50280, "time_step_rank": 48}')
    assert (c.family, c.d_model, c.n_layers, c.d_state, c.d_conv, c.expand, c.vocab_size) == ("mamba1", 768, 24, 16, 4, 2, 50280)
    assert c.tie_word_embeddings and not c.use_bias and c.use_conv_bias and c.rms_norm_eps == 1e-5


def test_parse_original_config():
    c = parse_config_json(b'{"d_model": 768, "n_layer": 24, "vocab_size": 50257}')
    assert (c.family, c.d_model, c.n_layers, c.d_state, c.d_conv, c.expand, c.vocab_size) == ("mamba1", 768, 24, 16, 4, 2, 50257)


def test_model_family_dispatch_and_errors():
    assert parse_config_json(_MIN_HF % "mamba").family == "mamba1"
    assert parse_config_json(_MIN_HF % "falcon_mamba").family == "mamba1"
    assert parse_config_json(_MIN_HF % "mamba2").family == "mamba2"
    assert parse_config_json('{"d_model":64,"n_layer":2,"vocab_size":100}').family == "mamba1"
    with pytest.raises(ValueError, match="unsupported model_type"):
        parse_config_json(_MIN_HF % "llama")
    with pytest.raises(ValueError, match="cannot detect model family"):
        parse_config_json('{"vocab_size": 5}')
    with pytest.raises(ValueError, match="time_step_rank mismatch"):
        parse_config_json('{"model_type":"mamba","hidden_size":768,"num_hidden_layers":24,"state_size":16,"conv_kernel":4,'
                          '"vocab_size":50280,"time_step_rank":999}')
    with pytest.raises(ValueError, match="missing|num_hidden_layers"):
        parse_config_json('{"model_type": "mamba", "hidden_size": 768}')
    with pytest.raises(ValueError, match="vocab_size"):
        parse_config_json('{"model_type":"mamba","hidden_size":64,"num_hidden_layers":2,"state_size":8,"conv_kernel":4}')
    with pytest.raises(ValueError, match="parse error"):
        parse_config_json(b"{not json")


def test_config_optional_fields():
    c = parse_config_json('{"model_type":"mamba","hidden_size":64,"num_hidden_layers":2,"state_size":8,"conv_kernel":4,"vocab_size":100,'
                          '"tie_word_embeddings":false,"use_conv_bias":false,"layer_norm_epsilon":1e-6}')
    assert not c.tie_word_embeddings and not c.use_conv_bias and c.rms_norm_eps == 1e-6
    c = parse_config_json('{"model_type":"mamba","hidden_size":64,"num_hidden_layers":2,"state_size":8,"conv_kernel":4,"vocab_size":100,'
                          '"rms_norm_eps":1e-4,"layer_norm_epsilon":1e-6}')
    assert c.rms_norm_eps == 1e-4     # rms_norm_eps wins over layer_norm_epsilon


# ---- serialize.rs ---------------------------------------------------------------------------------------

def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).ravel()


def test_native_round_trip_is_bit_exact(tmp_path):
    cfg = MambaConfig()
    w = MambaWeights.init(cfg, 128, 42)
    path = str(tmp_path / "model.safetensors")
    formats.save(path, w, cfg, 128)
    w2, cfg2, input_dim = formats.load(path)
    assert cfg2 == cfg and input_dim == 128
    assert (_bits(w.input_proj_w) == _bits(w2.input_proj_w)).all() and (_bits(w.norm_f_weight) == _bits(w2.norm_f_weight)).all()
    for a, b in zip(w.layers, w2.layers):
        for f in ("norm_weight", "in_proj_w", "conv1d_weight", "conv1d_bias", "x_proj_w", "dt_proj_w", "dt_proj_b", "a_log", "d_param", "out_proj_w"):
            assert (_bits(getattr(a, f)) == _bits(getattr(b, f))).all(), f


def test_native_file_carries_the_reference_names_shapes_and_metadata(tmp_path):
    from safetensors import safe_open
    cfg = MambaConfig(d_model=32, d_state=8, d_conv=4, expand=2, n_layers=2, scan_mode=ScanMode.SEQUENTIAL, rms_norm_eps=1e-6)
    path = str(tmp_path / "m.safetensors")
    formats.save(path, MambaWeights.init(cfg, 10, 1), cfg, 10)
    with safe_open(path, framework="np") as st:
        assert st.metadata()["config"] == ('{"d_model":32,"d_state":8,"d_conv":4,"expand":2,"n_layers":2,"input_dim":10,'
                                           '"scan_mode":"Sequential","rms_norm_eps":0.000001}')
        shapes = {k: tuple(st.get_slice(k).get_shape()) for k in st.keys()}
    want = {"input_proj.weight": (10, 32), "input_proj.bias": (32,), "norm_f.weight": (32,)}
    for i in range(2):
        want.update({f"layers.{i}.norm.weight": (32,), f"layers.{i}.in_proj.weight": (32, 128), f"layers.{i}.conv1d.weight": (64, 4),
                     f"layers.{i}.conv1d.bias": (64,), f"layers.{i}.x_proj.weight": (64, 18), f"layers.{i}.dt_proj.weight": (2, 64),
                     f"layers.{i}.dt_proj.bias": (64,), f"layers.{i}.a_log": (64, 8), f"layers.{i}.D": (64,),
                     f"layers.{i}.out_proj.weight": (64, 32)})
    assert shapes == want
    _, cfg2, _ = formats.load(path)
    assert cfg2.scan_mode == ScanMode.SEQUENTIAL and np.float32(cfg2.rms_norm_eps) == np.float32(1e-6)


def test_native_load_defaults_and_errors(tmp_path):
    from safetensors.numpy import save_file
    cfg = MambaConfig(d_model=16, d_state=4, d_conv=4, expand=2, n_layers=1)
    path = str(tmp_path / "m.safetensors")
    formats.save(path, MambaWeights.init(cfg, 16, 3), cfg, 16)
    from safetensors import safe_open
    with safe_open(path, framework="np") as st:
        tensors = {k: st.get_tensor(k) for k in st.keys()}
    # an older file without scan_mode / rms_norm_eps falls back to Auto and 1e-5 (serialize.rs:163-186)
    old = '{"d_model":16,"d_state":4,"d_conv":4,"expand":2,"n_layers":1,"input_dim":16}'
    save_file(tensors, path, metadata={"config": old})
    _, c, _ = formats.load(path)
    assert c.scan_mode == ScanMode.AUTO and c.rms_norm_eps == 1e-5
    save_file(tensors, path)
    with pytest.raises(ValueError, match="config"):
        formats.load(path)
    t2 = dict(tensors); del t2["layers.0.a_log"]
    save_file(t2, path, metadata={"config": old})
    with pytest.raises(ValueError, match="layers.0.a_log"):
        formats.load(path)
    t3 = dict(tensors); t3["layers.0.D"] = tensors["layers.0.D"].astype(np.float16)
    save_file(t3, path, metadata={"config": old})
    with pytest.raises(ValueError, match="F32"):
        formats.load(path)
    t4 = dict(tensors); t4["layers.0.D"] = tensors["layers.0.D"][:-1]
    save_file(t4, path, metadata={"config": old})
    with pytest.raises(ValueError, match="d_param"):
        formats.load(path)


def test_mamba3_native_round_trip(tmp_path):
    """mamba3_siso/serialize.rs:157-172, plus the file's names, shapes and metadata strings."""
    from safetensors import safe_open
    from mamba_rs_amd import Mamba3Config, Mamba3Weights
    cfg = Mamba3Config(d_model=32, n_layers=2)
    w = Mamba3Weights.init(cfg, 24, 42)
    path = str(tmp_path / "m3.safetensors")
    formats.save_mamba3(path, w, cfg, 24)
    w2, input_dim = formats.load_mamba3(path, cfg)
    assert input_dim == 24 and (_bits(w.input_proj_w) == _bits(w2.input_proj_w)).all() and (_bits(w.norm_f_weight) == _bits(w2.norm_f_weight)).all()
    for a, b in zip(w.layers, w2.layers):
        for f in ("norm_weight", "in_proj_w", "dt_bias", "b_norm_weight", "c_norm_weight", "b_bias", "c_bias", "d_param", "norm_gate_weight", "out_proj_w"):
            assert (_bits(getattr(a, f)) == _bits(getattr(b, f))).all(), f
    with safe_open(path, framework="np") as st:
        assert st.metadata() == {"d_model": "32", "d_state": "16", "expand": "2", "headdim": "16", "ngroups": "1", "n_layers": "2",
                                 "input_dim": "24", "rope_fraction": "0.5", "a_floor": "0.0001", "mamba_version": "3"}
        shapes = {k: tuple(st.get_slice(k).get_shape()) for k in st.keys()}
    nh, ip = cfg.nheads(), cfg.in_proj_out_dim()
    assert shapes["layers.1.in_proj.weight"] == (32, ip) and shapes["layers.0.b_bias"] == (nh, 16) and shapes["layers.0.D"] == (nh,)
    assert shapes["input_proj.weight"] == (24, 32) and shapes["layers.1.norm_gate.weight"] == (64,) and len(shapes) == 3 + 2 * 10
    with pytest.raises(ValueError, match="layers.2"):
        formats.load_mamba3(path, Mamba3Config(d_model=32, n_layers=3))
    with pytest.raises(ValueError, match="in_proj_w"):
        formats.load_mamba3(path, Mamba3Config(d_model=32, n_layers=2, d_state=32))


# ---- load.rs: the synthetic checkpoint of tests/hf_integration.rs ---------------------------------------

DM, DS, DC, EX, NL, VOCAB = 64, 16, 4, 2, 2, 256
DI, DR = DM * EX, -(-DM // 16)
XD = DR + 2 * DS


def rand_vec(n, seed):
    """xorshift64 fill of tests/hf_integration.rs:34-47."""
    s, out, mask = max(seed, 1), np.empty(n, np.float32), (1 << 64) - 1
    for i in range(n):
        s ^= (s << 13) & mask; s ^= s >> 7; s ^= (s << 17) & mask
        out[i] = np.float32(np.float32(s / float(mask) * 2.0 - 1.0) * np.float32(0.1))
    return out


def synthetic_tensors(include_lm_head):
    t = {"backbone.embeddings.weight": rand_vec(VOCAB * DM, 100).reshape(VOCAB, DM), "backbone.norm_f.weight": np.ones(DM, np.float32)}
    if include_lm_head:
        t["lm_head.weight"] = rand_vec(VOCAB * DM, 200).reshape(VOCAB, DM)
    for i in range(NL):
        sb, p = (i + 1) * 1000, f"backbone.layers.{i}"
        t[f"{p}.norm.weight"] = np.ones(DM, np.float32)
        t[f"{p}.mixer.in_proj.weight"] = rand_vec(2 * DI * DM, sb + 1).reshape(2 * DI, DM)
        t[f"{p}.mixer.conv1d.weight"] = rand_vec(DI * DC, sb + 2).reshape(DI, 1, DC)
        t[f"{p}.mixer.conv1d.bias"] = np.zeros(DI, np.float32)
        t[f"{p}.mixer.x_proj.weight"] = rand_vec(XD * DI, sb + 3).reshape(XD, DI)
        t[f"{p}.mixer.dt_proj.weight"] = rand_vec(DI * DR, sb + 4).reshape(DI, DR)
        t[f"{p}.mixer.dt_proj.bias"] = rand_vec(DI, sb + 5)
        t[f"{p}.mixer.A_log"] = (-np.log(np.arange(DI * DS, dtype=np.float32) + np.float32(1))).reshape(DI, DS)
        t[f"{p}.mixer.D"] = np.ones(DI, np.float32)
        t[f"{p}.mixer.out_proj.weight"] = rand_vec(DM * DI, sb + 6).reshape(DM, DI)
    return t


def write_synthetic_checkpoint(directory, include_lm_head=False, config_extra=None, tensors=None):
    from safetensors.numpy import save_file
    cfgj = {"model_type": "mamba", "hidden_size": DM, "num_hidden_layers": NL, "state_size": DS, "conv_kernel": DC, "expand": EX,
            "vocab_size": VOCAB, "time_step_rank": DR}
    cfgj.update(config_extra or {})
    with open(os.path.join(directory, "config.json"), "w") as fh:
        json.dump(cfgj, fh)
    tensors = synthetic_tensors(include_lm_head) if tensors is None else tensors
    save_file({k: np.ascontiguousarray(v) for k, v in tensors.items()}, os.path.join(directory, "model.safetensors"))
    return tensors


def test_load_synthetic_checkpoint_transposes_and_pads(tmp_path):
    t = write_synthetic_checkpoint(str(tmp_path))
    m = load_hf(str(tmp_path))
    assert (m.vocab_size, m.vocab_size_padded, m.cfg.d_model, m.cfg.n_layers, m.lm_head) == (VOCAB, 256, DM, NL, None)
    assert m.embed.shape == (256, DM) and (m.embed == t["backbone.embeddings.weight"]).all()
    assert m.weights.input_proj_w.size == 0
    for i, lw in enumerate(m.weights.layers):
        p = f"backbone.layers.{i}.mixer."
        # element [in, out] of ours is element [out, in] of the file
        assert lw.in_proj_w.shape == (DM, 2 * DI) and lw.in_proj_w[5, 7] == t[p + "in_proj.weight"][7, 5]
        assert (lw.in_proj_w == t[p + "in_proj.weight"].T).all()
        assert lw.x_proj_w.shape == (DI, XD) and (lw.x_proj_w == t[p + "x_proj.weight"].T).all()
        assert lw.dt_proj_w.shape == (DR, DI) and (lw.dt_proj_w == t[p + "dt_proj.weight"].T).all()
        assert lw.out_proj_w.shape == (DI, DM) and (lw.out_proj_w == t[p + "out_proj.weight"].T).all()
        assert lw.conv1d_weight.shape == (DI, DC) and (lw.conv1d_weight == t[p + "conv1d.weight"][:, 0, :]).all()
        assert (lw.a_log == t[p + "A_log"]).all() and (lw.dt_proj_b == t[p + "dt_proj.bias"]).all()
        assert lw.a_neg()[0, 0] < 0 and np.isfinite(lw.a_neg()).all()     # test_compute_a_neg_called
    m.weights.validate(m.cfg, m.cfg.d_model)


def test_untied_head_is_transposed_and_tied_config_drops_it(tmp_path):
    t = write_synthetic_checkpoint(str(tmp_path), include_lm_head=True, config_extra={"tie_word_embeddings": False})
    m = load_hf(str(tmp_path))
    assert m.lm_head.shape == (DM, VOCAB) and (m.lm_head == t["lm_head.weight"].T).all()
    write_synthetic_checkpoint(str(tmp_path), include_lm_head=True)         # tie_word_embeddings defaults to true
    assert load_hf(str(tmp_path)).lm_head is None
    write_synthetic_checkpoint(str(tmp_path), include_lm_head=False, config_extra={"tie_word_embeddings": False})
    with pytest.raises(ValueError, match="lm_head.weight not found"):
        load_hf(str(tmp_path))


def test_vocab_padding_and_original_key_names(tmp_path):
    t = synthetic_tensors(False)
    t["backbone.embedding.weight"] = t.pop("backbone.embeddings.weight")[:250]
    t["unrelated.tensor"] = np.zeros(3, np.float32)
    write_synthetic_checkpoint(str(tmp_path), config_extra={"vocab_size": 250}, tensors=t)
    m = load_hf(str(tmp_path))
    assert (m.vocab_size, m.vocab_size_padded) == (250, 256)
    assert (m.embed[:250] == t["backbone.embedding.weight"]).all() and (m.embed[250:] == 0).all()


def test_loader_errors(tmp_path):
    d = str(tmp_path)
    write_synthetic_checkpoint(d, config_extra={"use_bias": True})
    with pytest.raises(ValueError, match="use_bias"):
        load_hf(d)
    t = synthetic_tensors(False); del t["backbone.layers.1.mixer.D"]
    write_synthetic_checkpoint(d, tensors=t)
    with pytest.raises(ValueError, match="layer 1: missing field: d_param"):
        load_hf(d)
    t = synthetic_tensors(False); t["backbone.layers.2.mixer.D"] = np.ones(DI, np.float32)
    write_synthetic_checkpoint(d, tensors=t)
    with pytest.raises(ValueError, match="layer index 2"):
        load_hf(d)
    t = synthetic_tensors(False); t["backbone.layers.0.mixer.x_proj.weight"] = np.zeros((XD, DI - 1), np.float32)
    write_synthetic_checkpoint(d, tensors=t)
    with pytest.raises(ValueError, match="x_proj_w"):
        load_hf(d)
    t = synthetic_tensors(False); t["backbone.layers.0.mixer.D"] = np.ones(DI, np.int32)
    write_synthetic_checkpoint(d, tensors=t)
    with pytest.raises(ValueError, match="unsupported dtype"):
        load_hf(d)
    write_synthetic_checkpoint(d, config_extra={"model_type": "mamba2"})
    with pytest.raises(ValueError, match="Mamba-1"):
        load_hf(d)
    write_synthetic_checkpoint(d)
    os.remove(os.path.join(d, "model.safetensors"))
    with pytest.raises(ValueError, match="no model.safetensors"):
        load_hf(d)


def test_conv_bias_absent_when_config_says_so(tmp_path):
    t = synthetic_tensors(False)
    for i in range(NL):
        del t[f"backbone.layers.{i}.mixer.conv1d.bias"]
    write_synthetic_checkpoint(str(tmp_path), config_extra={"use_conv_bias": False}, tensors=t)
    m = load_hf(str(tmp_path))
    assert all((lw.conv1d_bias == 0).all() and lw.conv1d_bias.shape == (DI,) for lw in m.weights.layers)


@pytest.mark.parametrize("dtype,shards", [("float32", 1), ("bfloat16", 1), ("float16", 3), ("float32", 4)])
def test_save_hf_load_hf_round_trip(tmp_path, dtype, shards):
    """Writer -> reader over every storage dtype the loader widens (load.rs:231-250) and over sharded files
    (load.rs:253-290): f32 is bit-exact, 16-bit files come back as the rounded values."""
    import torch
    cfg = MambaConfig(d_model=48, d_state=8, d_conv=4, expand=2, n_layers=3, rms_norm_eps=1e-6)
    w = MambaWeights.random_lm(cfg, seed=9, std=0.1)
    rng = np.random.default_rng(1)
    vocab = 131
    embed = rng.standard_normal((vocab, 48)).astype(np.float32)
    head = rng.standard_normal((48, vocab)).astype(np.float32)
    save_hf(str(tmp_path), cfg, w, embed, vocab, dtype=dtype, lm_head=head, shards=shards)
    if shards > 1:
        assert os.path.exists(tmp_path / "model.safetensors.index.json") and not os.path.exists(tmp_path / "model.safetensors")
    m = load_hf(str(tmp_path))
    tdt = getattr(torch, dtype)
    rt = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(tdt).to(torch.float32).numpy()
    assert m.cfg == cfg and (m.vocab_size, m.vocab_size_padded) == (131, 192)
    assert (m.embed[:vocab] == rt(embed)).all() and (m.embed[vocab:] == 0).all() and (m.lm_head == rt(head)).all()
    for a, b in zip(w.layers, m.weights.layers):
        for f in ("norm_weight", "in_proj_w", "conv1d_weight", "conv1d_bias", "x_proj_w", "dt_proj_w", "dt_proj_b", "a_log", "d_param", "out_proj_w"):
            assert getattr(b, f).shape == getattr(a, f).shape and (getattr(b, f) == rt(getattr(a, f))).all(), f
