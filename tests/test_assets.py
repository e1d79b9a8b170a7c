"""Model assets: the safetensors tensor store, config.json and the GPT-2 weight-name
mapping (src/models/safetensors.rs, src/models/config.rs, src/models/gpt2/rust.rs:684-785).

Files are written here with the `safetensors` package (an independent writer of the
format) and by hand, byte by byte, for the malformed cases; the store under test is the
library's own reader."""
import json
import struct

import numpy as np
import pytest
from safetensors.numpy import save_file

import oracle
from helpers import assert_logits_close, numpy_gpt2_forward, small_cases
from puppygrad_amd import (Gpt2Config, Gpt2Error, Gpt2HipConfig, Gpt2Model, TensorStore,
                           load_weights, synth)

BLOCK_NAMES = {  # Gpt2BlockWeights field -> Hugging Face name (src/models/gpt2/rust.rs:719-750)
    "ln_1_g": "ln_1.weight", "ln_1_b": "ln_1.bias", "c_attn_w": "attn.c_attn.weight",
    "c_attn_b": "attn.c_attn.bias", "c_proj_w": "attn.c_proj.weight",
    "c_proj_b": "attn.c_proj.bias", "ln_2_g": "ln_2.weight", "ln_2_b": "ln_2.bias",
    "c_fc_w": "mlp.c_fc.weight", "c_fc_b": "mlp.c_fc.bias", "c_proj_mlp_w": "mlp.c_proj.weight",
    "c_proj_mlp_b": "mlp.c_proj.bias"}


def hf_tensors(cfg: Gpt2Config, w, prefix: str = "") -> dict:
    c, i = cfg.n_embd, cfg.n_inner
    shapes = {"ln_1_g": [c], "ln_1_b": [c], "c_attn_w": [c, 3 * c], "c_attn_b": [3 * c],
              "c_proj_w": [c, c], "c_proj_b": [c], "ln_2_g": [c], "ln_2_b": [c],
              "c_fc_w": [c, i], "c_fc_b": [i], "c_proj_mlp_w": [i, c], "c_proj_mlp_b": [c]}
    f = lambda a, s: np.ascontiguousarray(np.asarray(a, np.float32).reshape(s))
    out = {prefix + "wte.weight": f(w.wte, [cfg.vocab_size, c]),
           prefix + "wpe.weight": f(w.wpe, [cfg.n_positions, c]),
           prefix + "ln_f.weight": f(w.ln_f_g, [c]), prefix + "ln_f.bias": f(w.ln_f_b, [c])}
    for l, b in enumerate(w.blocks):
        for field, name in BLOCK_NAMES.items():
            out[f"{prefix}h.{l}.{name}"] = f(getattr(b, field), shapes[field])
    return out


def write_model_dir(path, cfg: Gpt2Config, w, prefix: str = "", extra: dict = None):
    path.mkdir(parents=True, exist_ok=True)
    save_file(hf_tensors(cfg, w, prefix), str(path / "model.safetensors"))
    hf = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "vocab_size": cfg.vocab_size,
          "n_positions": cfg.n_positions, "n_ctx": cfg.n_positions, "n_embd": cfg.n_embd,
          "n_layer": cfg.n_layer, "n_head": cfg.n_head, "n_inner": cfg.n_inner,
          "layer_norm_epsilon": cfg.layer_norm_epsilon, "activation_function": "gelu_new",
          "task_specific_params": {"text-generation": {"do_sample": True, "max_length": 50}}}
    hf.update(extra or {})
    (path / "config.json").write_text(json.dumps(hf, indent=2))
    return path


def same_config(a: Gpt2Config, b: Gpt2Config) -> bool:
    """Equal as the library holds them: layer_norm_epsilon is an f32 there."""
    key = lambda c: (c.vocab_size, c.n_positions, c.n_embd, c.n_layer, c.n_head, c.n_inner,
                     np.float32(c.layer_norm_epsilon))
    return key(a) == key(b)


def raw_file(path, header: dict, data: bytes, pad_to: int = 8, header_bytes: bytes = None):
    text = header_bytes if header_bytes is not None else json.dumps(header).encode()
    if pad_to:
        text += b" " * (-len(text) % pad_to)
    path.write_bytes(struct.pack("<Q", len(text)) + text + data)
    return path


# ---- the reference's own store tests (src/models/safetensors.rs:187-219) ----

def test_tensor_store_reads_required_and_optional_f32_tensors(tmp_path):
    values = np.array([[1.0, 2.5], [-3.0, 4.0]], np.float32)
    save_file({"weight": values}, str(tmp_path / "memory.safetensors"))
    store = TensorStore(tmp_path / "memory.safetensors")
    assert len(store) == 1
    got = store.required_f32("weight", [2, 2])
    assert got.dtype == np.float32 and got.tolist() == values.tolist()
    assert store.optional_f32("missing", [1]) is None
    assert store.optional_f32("weight", [2, 2]).tolist() == values.tolist()
    with pytest.raises(Gpt2Error) as e:
        store.required_f32("missing", [1])
    assert e.value.kind == "Asset" and "failed to read tensor missing" in str(e.value)


def test_tensor_store_validates_shape(tmp_path):
    save_file({"weight": np.zeros(1, np.float32)}, str(tmp_path / "m.safetensors"))
    store = TensorStore(tmp_path / "m.safetensors")
    with pytest.raises(Gpt2Error) as e:
        store.required_f32("weight", [2])
    assert e.value.kind == "InvalidWeights"
    assert "tensor weight shape [1] does not match expected [2]" in str(e.value)
    with pytest.raises(Gpt2Error, match=r"shape \[1\] does not match expected \[1, 1\]"):
        store.optional_f32("weight", [1, 1])


def test_tensor_store_validates_dtype(tmp_path):
    save_file({"half": np.zeros(4, np.float16), "ids": np.zeros(2, np.int64)},
              str(tmp_path / "m.safetensors"))
    store = TensorStore(tmp_path / "m.safetensors")
    with pytest.raises(Gpt2Error) as e:
        store.required_f32("half", [4])
    assert e.value.kind == "Asset" and "tensor half has dtype F16, expected F32" in str(e.value)
    with pytest.raises(Gpt2Error, match="tensor ids has dtype I64, expected F32"):
        store.required_f32("ids", [2])


def test_tensor_store_views_survive_the_store_object(tmp_path):
    a = synth.normal_f32(1000, 7, 0).reshape(10, 100)
    save_file({"a": a, "b": np.arange(6, dtype=np.float32)}, str(tmp_path / "m.safetensors"))
    view = TensorStore(tmp_path / "m.safetensors").required_f32("a", [10, 100])
    row = view[3]  # a derived view keeps the mapping alive as well
    del view
    assert np.array_equal(row, a[3])
    assert not row.flags.writeable


def test_tensor_store_reads_a_hand_written_file_whose_data_is_not_4_byte_aligned(tmp_path):
    vals = np.array([0.5, -1.25, 3.0e-7, 1.0e30, -0.0], np.float32)
    two = np.array([[7.0], [9.0]], np.float32)
    header = {"__metadata__": {"format": "pt", "note": "café \U0001F600 \"q\""},
              "x": {"dtype": "F32", "shape": [5], "data_offsets": [0, 20]},
              "z_empty": {"dtype": "F32", "shape": [0, 3], "data_offsets": [20, 20]},
              "y": {"dtype": "F32", "shape": [2, 1], "data_offsets": [20, 28]}}
    text = json.dumps(header).encode()  # ensure_ascii: exercises \u escapes and a surrogate pair
    if len(text) % 4 == 0:
        text += b" "
    path = raw_file(tmp_path / "odd.safetensors", None, vals.tobytes() + two.tobytes(), pad_to=0,
                    header_bytes=text)
    store = TensorStore(path)
    assert len(store) == 3
    assert store.required_f32("x", [5]).tobytes() == vals.tobytes()
    assert store.required_f32("y", [2, 1]).tolist() == two.tolist()
    assert store.required_f32("z_empty", [0, 3]).shape == (0, 3)  # an empty tensor shares its offset


@pytest.mark.parametrize("what", ["short", "huge_header", "header_past_end", "not_json", "not_object",
                                  "offset_past_end", "size_mismatch", "hole", "trailing_data",
                                  "unknown_dtype", "negative_dim"])
def test_tensor_store_rejects_malformed_files(tmp_path, what):
    path = tmp_path / f"{what}.safetensors"
    good = {"x": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}
    data = bytes(8)
    if what == "short":
        path.write_bytes(b"\x01\x00\x00")
    elif what == "huge_header":
        path.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    elif what == "header_past_end":
        path.write_bytes(struct.pack("<Q", 64) + b"{}")
    elif what == "not_json":
        raw_file(path, None, data, header_bytes=b'{"x": {"dtype": "F32", "shape": [2}')
    elif what == "not_object":
        raw_file(path, None, data, header_bytes=b"[1, 2, 3]")
    elif what == "offset_past_end":
        raw_file(path, {"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, data)
    elif what == "size_mismatch":
        raw_file(path, {"x": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, data)
    elif what == "hole":
        raw_file(path, {"x": {"dtype": "F32", "shape": [1], "data_offsets": [4, 8]}}, data)
    elif what == "trailing_data":
        raw_file(path, good, data + bytes(4))
    elif what == "unknown_dtype":
        raw_file(path, {"x": {"dtype": "F33", "shape": [2], "data_offsets": [0, 8]}}, data)
    elif what == "negative_dim":
        raw_file(path, {"x": {"dtype": "F32", "shape": [-2], "data_offsets": [0, 8]}}, data)
    with pytest.raises(Gpt2Error) as e:
        TensorStore(path)
    assert e.value.kind == "Asset"
    assert f"failed to parse safetensors file {path}" in str(e.value)


def test_tensor_store_reports_unreadable_files(tmp_path):
    with pytest.raises(Gpt2Error) as e:
        TensorStore(tmp_path / "nope.safetensors")
    assert e.value.kind == "Asset"
    assert f"failed to read safetensors file {tmp_path / 'nope.safetensors'}" in str(e.value)
    assert "No such file or directory" in str(e.value)
    with pytest.raises(Gpt2Error, match="failed to read safetensors file"):
        TensorStore(tmp_path)  # a directory


# ---- config.json (src/models/gpt2/rust.rs:684-711) ----

def test_load_config_reads_a_hugging_face_config(tmp_path):
    p = tmp_path / "config.json"
    p.write_text(json.dumps({
        "activation_function": "gelu_new", "architectures": ["GPT2LMHeadModel"], "attn_pdrop": 0.1,
        "bos_token_id": 50256, "embd_pdrop": 0.1, "eos_token_id": 50256, "initializer_range": 0.02,
        "layer_norm_epsilon": 1e-05, "model_type": "gpt2", "n_ctx": 1024, "n_embd": 768,
        "n_head": 12, "n_layer": 12, "n_positions": 1024, "resid_pdrop": 0.1,
        "summary_activation": None, "summary_first_dropout": 0.1, "summary_proj_to_labels": True,
        "summary_type": "cls_index", "summary_use_proj": True,
        "task_specific_params": {"text-generation": {"do_sample": True, "max_length": 50}},
        "vocab_size": 50257}))
    cfg = Gpt2Config.from_json_file(p)
    assert (cfg.vocab_size, cfg.n_positions, cfg.n_embd, cfg.n_layer, cfg.n_head) == \
        (50257, 1024, 768, 12, 12)
    assert cfg.n_inner == 3072 and cfg.layer_norm_epsilon == np.float32(1e-5)


def test_load_config_optional_fields(tmp_path):
    p = tmp_path / "config.json"
    base = {"vocab_size": 100, "n_embd": 8, "n_layer": 2, "n_head": 2}
    p.write_text(json.dumps({**base, "n_ctx": 32, "n_inner": None}))
    cfg = Gpt2Config.from_json_file(p)  # n_ctx stands in for n_positions; null n_inner -> 4C
    assert cfg.n_positions == 32 and cfg.n_inner == 32 and cfg.layer_norm_epsilon == np.float32(1e-5)
    p.write_text(json.dumps({**base, "n_positions": 16, "n_ctx": 32, "n_inner": 24,
                             "layer_norm_epsilon": 1e-6}))
    cfg = Gpt2Config.from_json_file(p)  # n_positions wins over n_ctx
    assert cfg.n_positions == 16 and cfg.n_inner == 24 and cfg.layer_norm_epsilon == np.float32(1e-6)


def test_load_config_errors(tmp_path):
    p = tmp_path / "config.json"
    base = {"vocab_size": 100, "n_embd": 8, "n_layer": 2, "n_head": 2}
    with pytest.raises(Gpt2Error) as e:
        Gpt2Config.from_json_file(p)
    assert e.value.kind == "Asset" and f"failed to read config {p}" in str(e.value)
    p.write_text(json.dumps(base))
    with pytest.raises(Gpt2Error) as e:
        Gpt2Config.from_json_file(p)
    assert e.value.kind == "InvalidConfig"
    assert "config must contain n_positions or n_ctx" in str(e.value)
    p.write_text(json.dumps({k: v for k, v in base.items() if k != "n_embd"} | {"n_ctx": 4}))
    with pytest.raises(Gpt2Error) as e:
        Gpt2Config.from_json_file(p)
    assert e.value.kind == "Asset" and "missing field `n_embd`" in str(e.value)
    p.write_text('{"vocab_size": 100, "n_embd": 8,')
    with pytest.raises(Gpt2Error) as e:
        Gpt2Config.from_json_file(p)
    assert e.value.kind == "Asset" and f"failed to parse config {p}" in str(e.value)
    p.write_text(json.dumps({**base, "n_ctx": 4, "n_layer": -1}))
    with pytest.raises(Gpt2Error, match="failed to parse config"):
        Gpt2Config.from_json_file(p)
    p.write_text(json.dumps({**base, "n_ctx": 4, "n_head": 3}))
    with pytest.raises(Gpt2Error) as e:  # validate() runs on the loaded config
        Gpt2Config.from_json_file(p)
    assert e.value.kind == "InvalidConfig" and "n_embd 8 must be divisible by n_head 3" in str(e.value)


# ---- weight names and layout (src/models/gpt2/rust.rs:713-785) ----

@pytest.mark.parametrize("prefix", ["", "transformer."])
def test_load_weights_maps_hugging_face_names(tmp_path, prefix):
    _, cfg, w, ids = small_cases()[2]
    d = write_model_dir(tmp_path / "m", cfg, w, prefix)
    assert same_config(Gpt2Config.from_json_file(d / "config.json"), cfg)
    got = load_weights(d / "model.safetensors", cfg)
    want = hf_tensors(cfg, w)
    assert np.array_equal(got.wte, want["wte.weight"]) and np.array_equal(got.wpe, want["wpe.weight"])
    assert np.array_equal(got.ln_f_g, want["ln_f.weight"])
    assert np.array_equal(got.ln_f_b, want["ln_f.bias"])
    for l, b in enumerate(got.blocks):
        for field, name in BLOCK_NAMES.items():
            assert np.array_equal(getattr(b, field), want[f"h.{l}.{name}"]), (l, field)
    # and the loaded tensors drive the model: the oracle on them equals float64 numpy on
    # the originals
    logits = oracle.Model(cfg, got).forward(ids)
    assert_logits_close(logits, numpy_gpt2_forward(cfg, w, ids))


def test_load_weights_errors(tmp_path):
    _, cfg, w, _ = small_cases()[0]
    tensors = hf_tensors(cfg, w)
    missing = {k: v for k, v in tensors.items() if k != "h.0.mlp.c_fc.bias"}
    save_file(missing, str(tmp_path / "missing.safetensors"))
    with pytest.raises(Gpt2Error) as e:
        load_weights(tmp_path / "missing.safetensors", cfg)
    assert e.value.kind == "Asset"
    assert "failed to read tensor transformer.h.0.mlp.c_fc.bias" in str(e.value)
    wrong = dict(tensors)
    wrong["h.0.attn.c_attn.weight"] = np.ascontiguousarray(tensors["h.0.attn.c_attn.weight"].T)
    save_file(wrong, str(tmp_path / "wrong.safetensors"))
    with pytest.raises(Gpt2Error) as e:  # [out,in] instead of the Conv1D [in,out]
        load_weights(tmp_path / "wrong.safetensors", cfg)
    assert e.value.kind == "InvalidWeights"
    assert "tensor h.0.attn.c_attn.weight shape [12, 4] does not match expected [4, 12]" in str(e.value)


def test_checkpoint_written_by_transformers_loads_and_matches_its_forward(tmp_path):
    """A GPT2LMHeadModel saved by the `transformers` library itself (its names carry the
    `transformer.` prefix and the tied lm_head is not stored): the oracle on the loaded
    tensors reproduces the library's own logits."""
    torch = pytest.importorskip("torch")
    transformers = pytest.importorskip("transformers")
    hf_cfg = transformers.GPT2Config(vocab_size=97, n_positions=24, n_embd=32, n_layer=2, n_head=4,
                                     n_inner=None, layer_norm_epsilon=1e-5,
                                     activation_function="gelu_new", resid_pdrop=0.0,
                                     embd_pdrop=0.0, attn_pdrop=0.0)
    torch.manual_seed(1234)
    model = transformers.GPT2LMHeadModel(hf_cfg).eval()
    with torch.no_grad():  # the default init leaves biases at 0 and LayerNorm at (1, 0)
        for name, p in model.named_parameters():
            if name.endswith("bias") or "ln_" in name:
                p.add_(0.1 * torch.randn_like(p))
    model.save_pretrained(str(tmp_path / "hf"), safe_serialization=True)
    cfg = Gpt2Config.from_json_file(tmp_path / "hf" / "config.json")
    assert (cfg.vocab_size, cfg.n_positions, cfg.n_embd, cfg.n_layer, cfg.n_head, cfg.n_inner) == \
        (97, 24, 32, 2, 4, 128)
    w = load_weights(tmp_path / "hf" / "model.safetensors", cfg)
    ids = [int(t) for t in synth.token_ids(19, 0x70C00303, 97)]
    with torch.no_grad():
        want = model(torch.tensor([ids])).logits[0].numpy()
    assert_logits_close(oracle.Model(cfg, w).forward(ids), want)


def test_from_dir_reports_asset_errors_before_any_device_work(tmp_path):
    _, cfg, w, _ = small_cases()[0]
    with pytest.raises(Gpt2Error) as e:
        Gpt2Model.from_dir(tmp_path / "absent")
    assert e.value.kind == "Asset" and "failed to read config" in str(e.value)
    d = write_model_dir(tmp_path / "m", cfg, w)
    (d / "model.safetensors").unlink()
    with pytest.raises(Gpt2Error, match="failed to read safetensors file"):
        Gpt2Model.from_dir(d)
    tensors = hf_tensors(cfg, w)
    tensors["wpe.weight"] = tensors["wpe.weight"][:-1]
    save_file(tensors, str(d / "model.safetensors"))
    with pytest.raises(Gpt2Error) as e:
        Gpt2Model.from_dir(d)
    assert e.value.kind == "InvalidWeights"
    assert "tensor wpe.weight shape [4, 4] does not match expected [5, 4]" in str(e.value)


# ---- the loaded model on the device ----

@pytest.mark.gpu
@pytest.mark.parametrize("prefix", ["", "transformer."])
def test_from_dir_model_equals_the_model_built_from_host_arrays(tmp_path, prefix):
    for name, cfg, w, ids in small_cases():
        d = write_model_dir(tmp_path / name, cfg, w, prefix)
        loaded = Gpt2Model.from_dir(d)
        assert same_config(loaded.config, cfg)
        direct = Gpt2Model.new(cfg, w)
        got = loaded.forward(ids).logits
        assert np.array_equal(got, direct.forward(ids).logits), name
        assert_logits_close(got, oracle.Model(cfg, w).forward(ids), what=name)
        c1, c2 = loaded.new_kv_cache(), direct.new_kv_cache()
        assert np.array_equal(loaded.prefill(ids, c1).to_host(), direct.prefill(ids, c2).to_host())
        n = min(5, cfg.n_positions - len(ids))
        assert loaded.generate_greedy(ids, n) == direct.generate_greedy(ids, n)


@pytest.mark.gpu
def test_from_dir_with_bf16_storage(tmp_path):
    _, cfg, w, ids = small_cases()[1]
    d = write_model_dir(tmp_path / "m", cfg, w)
    hip = Gpt2HipConfig(weight_storage=1)
    got = Gpt2Model.from_dir(d, hip).forward(ids).logits
    assert np.array_equal(got, Gpt2Model.new(cfg, w, hip).forward(ids).logits)
