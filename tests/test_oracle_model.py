"""Pins the oracle's full model: float64 numpy GPT-2 (matrix form, HF layout),
Hugging Face golden vectors, and the reference's own invariant tests
(src/models/gpt2/rust.rs:1865-2020)."""
import numpy as np
import pytest

import oracle
from helpers import assert_logits_close, load_golden, numpy_gpt2_forward, small_cases
from puppygrad_amd import synth


@pytest.mark.parametrize("case", small_cases(), ids=lambda c: c[0])
def test_forward_matches_float64_numpy(case):
    _, cfg, w, ids = case
    m = oracle.Model(cfg, w)
    got = m.forward(ids)
    want = numpy_gpt2_forward(cfg, w, ids)
    assert_logits_close(got, want, abs_tol=2e-5, rel_tol=1e-4)


@pytest.mark.parametrize("name", ["hf_c128_l2", "hf_c192_l3_h3", "hf_gpt2_small"])
def test_forward_matches_hf_golden(name):
    cfg, w, z = load_golden(name)
    ids = z["ids"]
    m = oracle.Model(cfg, w, oracle.rust_config(4))
    if cfg.vocab_size > 1000:
        cache = m.new_kv_cache()
        logits = m.prefill(ids, cache)[None]
        assert int(np.argmax(logits[0])) == int(z["argmax"])
    else:
        logits = m.forward(ids)
    got = logits[np.ix_(z["rows"] if cfg.vocab_size <= 1000 else [0], z["cols"])]
    assert_logits_close(got, z["logits"], abs_tol=3e-5, rel_tol=2e-4)


def test_tiny_fixture_closed_form_values():
    # tiny_weights is a closed form (rust.rs:2094-2121); spot-check what the oracle was given
    cfg = synth.tiny_config()
    w = synth.tiny_weights(cfg)
    np.testing.assert_allclose(w.wte[:4], np.array([0, -6, 11, 5]) * np.float32(0.03), rtol=1e-6)
    assert w.blocks[0].c_attn_w.size == 4 * 12 and w.blocks[0].c_proj_mlp_w.size == 8 * 4


def test_validates_weight_shapes():
    # rust.rs:1865-1873
    cfg = synth.tiny_config()
    w = synth.tiny_weights(cfg)
    w.wte = w.wte[:-1]
    with pytest.raises(oracle.OracleError) as e:
        oracle.Model(cfg, w)
    assert "wte len" in str(e.value)


def test_forward_returns_logits_for_each_position():
    # rust.rs:1875-1886
    cfg = synth.tiny_config()
    out = oracle.Model(cfg, synth.tiny_weights(cfg)).forward([1, 2, 3])
    assert out.shape == (3, cfg.vocab_size) and np.isfinite(out).all()


def test_greedy_generation_appends_tokens_until_context_limit():
    # rust.rs:1888-1898
    cfg = synth.tiny_config()
    tokens = oracle.Model(cfg, synth.tiny_weights(cfg)).generate_greedy([0, 1], 10)
    assert len(tokens) == cfg.n_positions and tokens[:2] == [0, 1]
    assert all(t < cfg.vocab_size for t in tokens)


@pytest.mark.parametrize("case", small_cases(), ids=lambda c: c[0])
def test_cached_prefill_matches_full_forward_last_logits(case):
    # rust.rs:1900-1913 (1e-5)
    _, cfg, w, ids = case
    m = oracle.Model(cfg, w)
    full = m.forward(ids)
    cache = m.new_kv_cache()
    cached = m.prefill(ids, cache)
    assert cache.seq_len == len(ids)
    np.testing.assert_allclose(cached, full[-1], atol=1e-5, rtol=0)


def test_kv_index_layout_against_full_sequence_qkv():
    # kv_index (rust.rs:1851-1855): [head][position][head_dim]; brute force from numpy
    _, cfg, w, ids = small_cases()[1]
    m = oracle.Model(cfg, w)
    cache = m.new_kv_cache()
    m.prefill(ids, cache)
    C, H, hd, T = cfg.n_embd, cfg.n_head, cfg.head_dim(), len(ids)
    f = lambda a, *s: np.asarray(a, np.float64).reshape(*s)
    x = f(w.wte, -1, C)[np.asarray(ids)] + f(w.wpe, -1, C)[:T]
    b = w.blocks[0]
    mu, var = x.mean(-1, keepdims=True), x.var(-1, keepdims=True)
    n = (x - mu) / np.sqrt(var + cfg.layer_norm_epsilon) * f(b.ln_1_g, C) + f(b.ln_1_b, C)
    qkv = n @ f(b.c_attn_w, C, 3 * C) + f(b.c_attn_b, 3 * C)
    k = qkv[:, C:2 * C].reshape(T, H, hd).transpose(1, 0, 2)
    v = qkv[:, 2 * C:].reshape(T, H, hd).transpose(1, 0, 2)
    np.testing.assert_allclose(cache.read_layer(0, 0)[:, :T], k, atol=1e-5)
    np.testing.assert_allclose(cache.read_layer(0, 1)[:, :T], v, atol=1e-5)
    assert not cache.read_layer(0, 0)[:, T:].any()  # zero-initialised beyond seq_len


def test_cached_greedy_generation_matches_full_generation():
    # rust.rs:1915-1925, 1944-1954
    cfg = synth.tiny_config()
    m = oracle.Model(cfg, synth.tiny_weights(cfg))
    assert m.generate([0, 1], 3) == m.generate_greedy([0, 1], 3)


def test_threaded_generation_matches_single_threaded():
    # rust.rs:1969-1995 (threads=3 vs 1) plus a model big enough to take the pooled paths
    cfg = synth.tiny_config()
    w = synth.tiny_weights(cfg)
    assert (oracle.Model(cfg, w, oracle.rust_config(3)).generate([0, 1], 3)
            == oracle.Model(cfg, w, oracle.rust_config(1)).generate([0, 1], 3))
    _, cfg, w, ids = small_cases()[1]
    rc = oracle.rust_config(3, dense_parallel_threshold=1024, attention_head_parallel_threshold=64)
    a, b = oracle.Model(cfg, w, rc), oracle.Model(cfg, w, oracle.rust_config(1))
    np.testing.assert_array_equal(a.forward(ids), b.forward(ids))
    ca, cb = a.new_kv_cache(), b.new_kv_cache()
    np.testing.assert_array_equal(a.prefill(ids, ca), b.prefill(ids, cb))


def test_cache_contract_and_errors():
    # rust.rs:1956-1967 and the error strings at 950-962, 1029-1051
    cfg = synth.tiny_config()
    m = oracle.Model(cfg, synth.tiny_weights(cfg))
    cache = m.new_kv_cache()
    cache.seq_len = 2
    assert cache.seq_len == 2 and cache.max_seq_len == cfg.n_positions
    cache.clear()
    assert cache.seq_len == 0
    with pytest.raises(oracle.OracleError, match="input_ids must not be empty"):
        m.prefill([], cache)
    with pytest.raises(oracle.OracleError, match="exceeds n_positions"):
        m.prefill([0] * 6, cache)
    with pytest.raises(oracle.OracleError, match="exceeds vocab_size"):
        m.forward_one(8, cache)
    m.prefill([0, 1, 2, 3, 4], cache)
    with pytest.raises(oracle.OracleError, match="cache is full at seq_len 5"):
        m.forward_one(1, cache)


def test_stream_loop_semantics():
    # rust.rs:495-531: EOS tested before the push, stop at n_positions, last forward skipped
    cfg = synth.tiny_config()
    m = oracle.Model(cfg, synth.tiny_weights(cfg))
    plain, st, _, _ = m.stream_token_ids_with_stats([0, 1], 10, None)
    assert len(plain) == cfg.n_positions and st.generated_tokens == 3
    assert plain == m.generate([0, 1], 10)
    first = plain[2]
    toks, st, _, _ = m.stream_token_ids_with_stats([0, 1], 10, first)
    assert toks == [0, 1] and st.generated_tokens == 0
    toks, st, logits, gap = m.stream_token_ids_with_stats([0, 1], 2, None, want_logits=True)
    assert toks == plain[:4] and logits.shape == (2, cfg.vocab_size) and (gap >= 0).all()
    with pytest.raises(oracle.OracleError, match="outside vocab_size"):
        m.stream_token_ids_with_stats([0, 1], 2, 8)
