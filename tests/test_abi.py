"""CPU-only checks of the C ABI: the library loads, exports every symbol the
header declares, and its host-side validation reproduces the reference's error
strings before any device work (src/models/gpt2/rust.rs:60-95, 1279-1343)."""
import ctypes as C
import re
from pathlib import Path

import numpy as np
import pytest

from puppygrad_amd import Gpt2Config, Gpt2Error, Gpt2Model, TextGenerationConfig, _lib, synth

HEADER = Path(__file__).resolve().parents[1] / "include" / "puppygrad_hip.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(pg_[a-z0-9_]+)\s*\(", text)) - {"pg_on_token"})


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_functions()
    assert len(names) >= 35
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names  # the ctypes table covers the header exactly


def test_config_validation_messages():
    w = synth.tiny_weights(synth.tiny_config())
    for field, msg in [("vocab_size", "vocab_size must be > 0"), ("n_positions", "n_positions must be > 0"),
                       ("n_embd", "n_embd must be > 0"), ("n_layer", "n_layer must be > 0"),
                       ("n_head", "n_head must be > 0"), ("n_inner", "n_inner must be > 0")]:
        cfg = synth.tiny_config()
        setattr(cfg, field, 0)
        with pytest.raises(Gpt2Error) as e:
            Gpt2Model.new(cfg, w)
        assert e.value.kind == "InvalidConfig" and msg in str(e.value)
    cfg = synth.tiny_config()
    cfg.n_head = 3
    with pytest.raises(Gpt2Error, match="n_embd 4 must be divisible by n_head 3"):
        Gpt2Model.new(cfg, w)
    cfg = synth.tiny_config()
    cfg.layer_norm_epsilon = 0.0
    with pytest.raises(Gpt2Error, match="layer_norm_epsilon must be > 0"):
        Gpt2Model.new(cfg, w)


def test_weight_validation_messages():
    cfg = synth.tiny_config()
    w = synth.tiny_weights(cfg)
    w.wte = w.wte[:-1]
    with pytest.raises(Gpt2Error) as e:
        Gpt2Model.new(cfg, w)
    assert e.value.kind == "InvalidWeights"
    assert "wte len 31 does not match expected 32" in str(e.value)
    w = synth.tiny_weights(cfg)
    w.blocks[0].c_fc_b = np.zeros(7, np.float32)
    with pytest.raises(Gpt2Error, match=r"blocks\[0\]\.c_fc_b len 7 does not match expected 8"):
        Gpt2Model.new(cfg, w)
    w = synth.tiny_weights(cfg)
    w.blocks = []
    with pytest.raises(Gpt2Error, match="blocks len 0 does not match n_layer 1"):
        Gpt2Model.new(cfg, w)


def test_sampling_validation_and_rng_known_answers():
    with pytest.raises(Gpt2Error, match="generation top_p must be finite and in"):
        TextGenerationConfig(1, top_p=2.0).validate()
    with pytest.raises(Gpt2Error, match="generation temperature"):
        TextGenerationConfig(1, temperature=float("nan")).validate()
    with pytest.raises(Gpt2Error, match="generation top_k must be > 0"):
        TextGenerationConfig(1, top_k=0).validate()
    with pytest.raises(Gpt2Error, match="generation repeat_penalty"):
        TextGenerationConfig(1, repeat_penalty=-1.0).validate()
    TextGenerationConfig(1, temperature=0.5, top_p=1.0, top_k=3).validate()
    lib = _lib.load()
    r = _lib.pg_rng_state()
    lib.pg_rng_seed(C.byref(r), 299792458)
    assert [lib.pg_rng_next_u64(C.byref(r)) for _ in range(3)] == [
        0x2788DF83E85DDB82, 0x8D4AF85AB3C903F9, 0xE889F1995D0FFA75]
    lib.pg_rng_seed(C.byref(r), 299792458)
    assert lib.pg_rng_next_unit_f64(C.byref(r)) == 0.1544322678604354


def test_synth_stream_is_counter_based_and_normal():
    a = synth.normal_f32(1000, 42, 0)
    b = synth.normal_f32(400, 42, 600)
    np.testing.assert_array_equal(a[600:], b)          # `first` indexes one stream
    big = synth.normal_f32(1 << 18, 7, 0)              # threaded path
    np.testing.assert_array_equal(big[:1000], synth.normal_f32(1000, 7, 0))
    assert abs(float(big.mean())) < 2e-4 and abs(float(big.std()) - 0.02) < 2e-4
    # Box-Muller from draws 2i, 2i+1 of splitmix64, restated with python integers
    M, G = (1 << 64) - 1, 0x9E3779B97F4A7C15

    def draw(seed, j):
        v = ((seed ^ G) + (j + 1) * G) & M
        v = ((v ^ (v >> 30)) * 0xBF58476D1CE4E5B9) & M
        v = ((v ^ (v >> 27)) * 0x94D049BB133111EB) & M
        return v ^ (v >> 31)

    for i in (0, 1, 999):
        u1 = ((draw(42, 2 * i) >> 11) + 1) / 2.0 ** 53
        u2 = (draw(42, 2 * i + 1) >> 11) / 2.0 ** 53
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2 * np.pi * u2)
        assert abs(float(a[i]) - z * 0.02) < 1e-9
    ids = synth.token_ids(5, 3, 50257)
    assert [int(t) for t in ids] == [draw(3, j) % 50257 for j in range(5)]


def test_no_device_is_a_loud_backend_error(has_gpu):
    if has_gpu:
        pytest.skip("a GPU is present")
    cfg = synth.tiny_config()
    with pytest.raises(Gpt2Error) as e:
        Gpt2Model.new(cfg, synth.tiny_weights(cfg))
    assert e.value.kind == "Backend" and "no HIP device" in str(e.value)
