"""The HIP backend behind the reference's model API: the reference's own GPT-2
unit tests (src/models/gpt2/rust.rs:1865-2020) re-run on it, plus logit parity
with the oracle and the Hugging Face golden vectors."""
import numpy as np
import pytest

import oracle
from helpers import ABS_TOL, REL_TOL, assert_logits_close, load_golden, small_cases
from puppygrad_amd import (Gpt2Error, Gpt2Model, LogitsSampler,
                           TextGenerationConfig, generate, synth)

pytestmark = pytest.mark.gpu


def tiny():
    cfg = synth.tiny_config()
    return cfg, Gpt2Model.new(cfg, synth.tiny_weights(cfg))


def test_validates_weight_shapes():
    cfg = synth.tiny_config()
    w = synth.tiny_weights(cfg)
    w.wte = w.wte[:-1]
    with pytest.raises(Gpt2Error) as e:
        Gpt2Model.new(cfg, w)
    assert "wte len" in str(e.value) and e.value.kind == "InvalidWeights"


def test_forward_returns_logits_for_each_position():
    cfg, model = tiny()
    out = model.forward([1, 2, 3])
    assert out.seq_len == 3 and out.vocab_size == cfg.vocab_size
    assert out.logits.shape == (3, cfg.vocab_size) and np.isfinite(out.logits).all()


def test_greedy_generation_appends_tokens_until_context_limit():
    cfg, model = tiny()
    tokens = model.generate_greedy([0, 1], 10)
    assert len(tokens) == cfg.n_positions and tokens[:2] == [0, 1]
    assert all(t < cfg.vocab_size for t in tokens)


def test_cached_prefill_matches_full_forward_last_logits():
    cfg, model = tiny()
    full = model.forward([1, 2, 3])
    cache = model.new_kv_cache()
    cached = model.prefill([1, 2, 3], cache).to_host()
    assert cache.seq_len == 3
    np.testing.assert_allclose(cached, full.last_logits(), atol=1e-5, rtol=0)


def test_cached_greedy_generation_matches_full_generation():
    _, model = tiny()
    assert model.generate_greedy_cached([0, 1], 3) == model.generate_greedy([0, 1], 3)


def test_streams_generated_tokens_in_order():
    _, model = tiny()
    streamed = []
    tokens = model.stream_greedy_tokens([0, 1], 3, streamed.append)
    assert tokens[:2] == [0, 1] and streamed == tokens[2:]


def test_implements_generic_autoregressive_decoder():
    _, model = tiny()
    assert generate(model, [0, 1], 3, lambda _t: None) == model.generate_greedy_cached([0, 1], 3)


def test_gpt2_cache_exposes_generic_kv_cache_contract():
    cfg, model = tiny()
    cache = model.new_kv_cache()
    cache.seq_len = 2
    assert cache.seq_len == 2 and cache.max_seq_len == cfg.n_positions
    cache.clear()
    assert cache.seq_len == 0


def test_tokens_match_oracle_on_tiny():
    cfg, model = tiny()
    ref = oracle.Model(cfg, synth.tiny_weights(cfg))
    assert model.generate_greedy_cached([0, 1], 3) == ref.generate([0, 1], 3)
    toks, stats = model.stream_token_ids_with_stats([0, 1], TextGenerationConfig(10))
    want, st, _, _ = ref.stream_token_ids_with_stats([0, 1], 10, None)
    assert toks == want and stats.generated_tokens == st.generated_tokens == 3


def test_error_surface():
    cfg, model = tiny()
    cache = model.new_kv_cache()
    with pytest.raises(Gpt2Error, match="input_ids must not be empty"):
        model.prefill([], cache)
    with pytest.raises(Gpt2Error, match="exceeds n_positions"):
        model.prefill([0] * 6, cache)
    with pytest.raises(Gpt2Error, match="at index 1 exceeds vocab_size"):
        model.prefill([0, 8], cache)
    with pytest.raises(Gpt2Error, match="exceeds vocab_size"):
        model.forward_one(8, cache)
    model.prefill([0, 1, 2, 3, 4], cache)
    with pytest.raises(Gpt2Error, match="cache is full at seq_len 5"):
        model.forward_one(1, cache)
    other = Gpt2Model.new(synth.Gpt2Config(vocab_size=8, n_positions=6, n_embd=4, n_layer=1, n_head=2),
                          synth.random_weights(synth.Gpt2Config(vocab_size=8, n_positions=6, n_embd=4,
                                                                n_layer=1, n_head=2), 1))
    with pytest.raises(Gpt2Error, match="cache max_seq_len 5 does not match n_positions 6"):
        other.forward_one(1, cache)
    bad = synth.tiny_config()
    bad.n_head = 3
    with pytest.raises(Gpt2Error, match="must be divisible by n_head"):
        Gpt2Model.new(bad, synth.tiny_weights(synth.tiny_config()))
    with pytest.raises(Gpt2Error, match="outside vocab_size"):
        model.stream_token_ids_with_stats([0, 1], TextGenerationConfig(2, eos_token_id=8))
    with pytest.raises(Gpt2Error, match="top_p"):
        model.stream_token_ids_with_stats([0, 1], TextGenerationConfig(2, top_p=2.0))


@pytest.mark.parametrize("case", small_cases(), ids=lambda c: c[0])
def test_logits_match_oracle_small(case):
    _, cfg, w, ids = case
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w)
    assert_logits_close(model.forward(ids).logits, ref.forward(ids))
    cache, rcache = model.new_kv_cache(), ref.new_kv_cache()
    assert_logits_close(model.prefill(ids, cache).to_host(), ref.prefill(ids, rcache))
    for tok in [1, 0, 5]:
        if cache.seq_len >= cfg.n_positions:
            break
        assert_logits_close(model.forward_one(tok, cache).to_host(), ref.forward_one(tok, rcache))
    for layer in range(cfg.n_layer):  # K/V cache layout is the reference's kv_index
        for which in (0, 1):
            np.testing.assert_allclose(cache.read_layer(layer, which)[:, :cache.seq_len],
                                       rcache.read_layer(layer, which)[:, :rcache.seq_len],
                                       atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("name", ["hf_c128_l2", "hf_c192_l3_h3", "hf_gpt2_small"])
def test_logits_match_hf_golden(name):
    cfg, w, z = load_golden(name)
    model = Gpt2Model.new(cfg, w)
    ids = z["ids"]
    if cfg.vocab_size > 1000:
        cache = model.new_kv_cache()
        logits = model.prefill(ids, cache)
        assert model.select_next_token(logits) == int(z["argmax"])
        got = logits.to_host()[z["cols"]][None]
    else:
        got = model.forward(ids).logits[np.ix_(z["rows"], z["cols"])]
    assert_logits_close(got, z["logits"])


def long_cases():
    """Prompts long enough (>= 16 tokens) to take the GEMM prefill / forward path."""
    out = []
    cfg = synth.Gpt2Config(vocab_size=211, n_positions=96, n_embd=128, n_layer=2, n_head=2)
    out.append(("c128_T67", cfg, synth.random_weights(cfg, 0x5EED0211, perturb=True),
                list(synth.token_ids(67, 0x70C00211, 211))))
    cfg = synth.Gpt2Config(vocab_size=300, n_positions=64, n_embd=48, n_layer=2, n_head=3, n_inner=112)
    out.append(("hd16_T40", cfg, synth.random_weights(cfg, 0x5EED0212, std=0.08, perturb=True),
                list(synth.token_ids(40, 0x70C00212, 300))))
    cfg = synth.Gpt2Config(vocab_size=97, n_positions=160, n_embd=192, n_layer=1, n_head=3)
    out.append(("c192_T160", cfg, synth.random_weights(cfg, 0x5EED0213, perturb=True),
                list(synth.token_ids(160, 0x70C00213, 97))))
    # 124M's layer shapes at 512 tokens: more 64x64 tiles than CUs with a partial last round
    # (c_attn 288, c_fc 384: the tail-split form with BIAS and GELU epilogues), split-K for the
    # projections back to n_embd, and attention blocks whose eight wavefronts get two key
    # tiles each
    cfg = synth.Gpt2Config(vocab_size=97, n_positions=512, n_embd=768, n_layer=1, n_head=12)
    out.append(("c768_T512", cfg, synth.random_weights(cfg, 0x5EED0214, perturb=True),
                list(synth.token_ids(512, 0x70C00214, 97))))
    return out


@pytest.mark.parametrize("case", long_cases(), ids=lambda c: c[0])
def test_gemm_prefill_and_forward_match_oracle(case):
    from puppygrad_amd import Gpt2HipConfig
    _, cfg, w, ids = case
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w)
    want_all = ref.forward(ids)
    assert_logits_close(model.forward(ids).logits, want_all)
    cache, rcache = model.new_kv_cache(), ref.new_kv_cache()
    assert_logits_close(model.prefill(ids, cache).to_host(), ref.prefill(ids, rcache))
    assert cache.seq_len == len(ids)
    for layer in range(cfg.n_layer):  # the GEMM path fills the cache in the reference's layout
        for which in (0, 1):
            np.testing.assert_allclose(cache.read_layer(layer, which)[:, :len(ids)],
                                       rcache.read_layer(layer, which)[:, :len(ids)],
                                       atol=2e-5, rtol=1e-4)
    if cache.seq_len < cfg.n_positions:  # decode continues from a GEMM-filled cache
        assert_logits_close(model.forward_one(3, cache).to_host(), ref.forward_one(3, rcache))
    # token-by-token prefill (the reference's own order) gives the same logits
    tok_model = Gpt2Model.new(cfg, w, Gpt2HipConfig(prefill_path=1))
    c2 = tok_model.new_kv_cache()
    assert_logits_close(tok_model.prefill(ids, c2).to_host(), want_all[-1])


@pytest.mark.parametrize("n_embd,n_head,n_prompt", [(768, 12, 30), (1024, 16, 140), (1280, 20, 60), (1600, 25, 200)])
def test_persistent_decode_every_width_matches_oracle(n_embd, n_head, n_prompt):
    """The four GPT-2 widths the persistent decode kernel is built for (small, medium, large,
    XL), f32 rows: single forwards and a multi-token launch against the oracle."""
    cfg = synth.Gpt2Config(vocab_size=300, n_positions=256, n_embd=n_embd, n_layer=2, n_head=n_head)
    w = synth.random_weights(cfg, 0x5EED0220 + n_head, perturb=True)
    ids = list(synth.token_ids(n_prompt, 0x70C00220, cfg.vocab_size))
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(8))
    assert "decode=persistent" in model.describe()
    cache, rcache = model.new_kv_cache(), ref.new_kv_cache()
    assert_logits_close(model.prefill(ids, cache).to_host(), ref.prefill(ids, rcache))
    rlog = None
    for tok in (7, 123, 42):
        rlog = ref.forward_one(tok, rcache)
        assert_logits_close(model.forward_one(tok, cache).to_host(), rlog)
    got, _ = model.decode_greedy(cache, 6)
    want, clear = [], True
    for i in range(6):
        top = np.sort(rlog)[-2:]
        clear = clear and (top[1] - top[0]) > 2 * (ABS_TOL + REL_TOL * abs(float(top[1])))
        want.append(oracle.argmax_logits(rlog))
        if i < 5:
            rlog = ref.forward_one(want[-1], rcache)
    assert len(got) == 6
    if clear:
        assert got == want


@pytest.mark.parametrize("n_prompt", [100, 1500, 2750])
def test_persistent_decode_split_counts_match_oracle(n_prompt):
    """The persistent decode kernel picks the number of key splits per head from the position:
    one split and no merge hop up to 128 keys (prompt 100), several with the merge done by
    workgroups that hold no attention item (prompt 1500: 12 splits, 144 items), and beyond one
    item per workgroup with the merge by the head's first split (prompt 2750: 22 splits, 264
    items on 256 workgroups).  One layer keeps the oracle cheap at these lengths."""
    cfg = synth.Gpt2Config(vocab_size=300, n_positions=4096, n_embd=768, n_layer=1, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0215, perturb=True)
    ids = list(synth.token_ids(n_prompt, 0x70C00215, cfg.vocab_size))
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(8))
    assert "decode=persistent" in model.describe()
    cache, rcache = model.new_kv_cache(), ref.new_kv_cache()
    assert_logits_close(model.prefill(ids, cache).to_host(), ref.prefill(ids, rcache))
    rlog = None
    for tok in (7, 123, 42):  # teacher-forced steps through the persistent kernel
        rlog = ref.forward_one(tok, rcache)
        assert_logits_close(model.forward_one(tok, cache).to_host(), rlog)
    got, _ = model.decode_greedy(cache, 6)  # five forwards in one launch
    want, clear = [], True
    for i in range(6):
        top = np.sort(rlog)[-2:]
        clear = clear and (top[1] - top[0]) > 2 * (ABS_TOL + REL_TOL * abs(float(top[1])))
        want.append(oracle.argmax_logits(rlog))
        if i < 5:
            rlog = ref.forward_one(want[-1], rcache)
    assert len(got) == 6
    if clear:  # no near-tie on the way: the ids are the oracle's
        assert got == want


def test_sampler_on_device_logits_matches_oracle():
    _, cfg, w, ids = small_cases()[1]
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w)
    cache, rcache = model.new_kv_cache(), ref.new_kv_cache()
    logits = model.prefill(ids, cache)
    rlogits = ref.prefill(ids, rcache)
    for kw in [dict(), dict(repeat_penalty=1.7), dict(temperature=0.9), dict(temperature=0.7, top_k=5),
               dict(temperature=1.1, top_p=0.8), dict(temperature=0.8, top_k=20, top_p=0.5, repeat_penalty=1.3)]:
        for seed in (1, 299792458):
            g = TextGenerationConfig(1, seed=seed, **kw)
            got = LogitsSampler(seed).select_next_token(logits, ids, g)
            want = oracle.LogitsSampler(seed).select_next_token(
                rlogits, ids, oracle.sampling(seed=seed, **kw))
            assert got == want, (kw, seed)


def test_sampler_with_tied_logits_keeps_the_stable_order():
    """Tokens with identical wte rows have bit-identical logits.  The reference sorts the
    candidates stably (generation.rs:311-312), so among ties the lower id ranks first and
    top_k may cut through a group of ties: the library's sampler, fed its own device
    logits, must pick what the oracle's sampler picks on those same values."""
    _, cfg, w, ids = small_cases()[1]
    wte = np.asarray(w.wte, np.float32).reshape(cfg.vocab_size, cfg.n_embd).copy()
    for i in range(cfg.vocab_size):
        wte[i] = wte[i % 7]  # seven distinct rows: 18-19 exact ties each
    w.wte = wte.reshape(-1)
    model = Gpt2Model.new(cfg, w)
    cache = model.new_kv_cache()
    logits = model.prefill(ids, cache)
    host = logits.to_host()
    assert len(np.unique(host)) <= 7
    cases = [dict(temperature=0.9, top_k=3), dict(temperature=1.3, top_k=20), dict(temperature=0.7, top_k=25, top_p=0.9),
             dict(temperature=1.0, top_k=1), dict(temperature=1.0, top_k=19), dict(temperature=1.0, top_k=130),
             dict(temperature=1.0, top_k=131), dict(temperature=1.1, top_k=500), dict(temperature=0.8, top_p=0.6),
             dict(temperature=1.0), dict(temperature=1.0, top_k=40, repeat_penalty=1.5),
             dict(temperature=0.6, top_k=7, repeat_penalty=3.0, repeat_last_n=5),
             dict(temperature=2.0, top_k=60, repeat_penalty=0.5, repeat_last_n=1000)]
    for kw in cases:
        for seed in (1, 2, 3, 299792458):
            g = TextGenerationConfig(1, seed=seed, **kw)
            got = LogitsSampler(seed).select_next_token(logits, ids, g)
            want = oracle.LogitsSampler(seed).select_next_token(host, ids, oracle.sampling(seed=seed, **kw))
            assert got == want, (kw, seed)


def test_sampler_over_a_large_vocabulary_with_ties():
    """More than 4096 candidates: without top_k the host orders the whole row (a stable radix
    sort on the values' integer image); with top_k the device picks the candidates.  Rows of
    wte are repeated so that the order among exact ties matters."""
    cfg = synth.Gpt2Config(vocab_size=6011, n_positions=32, n_embd=128, n_layer=1, n_head=2)
    w = synth.random_weights(cfg, 0x5EED0230, perturb=True)
    wte = np.asarray(w.wte, np.float32).reshape(cfg.vocab_size, cfg.n_embd).copy()
    for i in range(cfg.vocab_size):
        wte[i] = wte[i % 997]  # six or seven exact ties per value
    wte[11] = np.inf           # and a few non-finite logits
    wte[4999] = -np.inf
    w.wte = wte.reshape(-1)
    ids = [int(t) for t in synth.token_ids(9, 0x70C00230, 997) if t not in (11,)]
    model = Gpt2Model.new(cfg, w)
    cache = model.new_kv_cache()
    logits = model.prefill(ids, cache)
    host = logits.to_host()
    assert len(np.unique(host[np.isfinite(host)])) <= 997
    for kw in [dict(temperature=1.0), dict(temperature=0.7, top_p=0.9), dict(temperature=1.5, top_p=0.999),
               dict(temperature=1.0, repeat_penalty=1.3), dict(temperature=1.0, top_k=5000),
               dict(temperature=1.0, top_k=4096), dict(temperature=0.9, top_k=300, top_p=0.95),
               dict(temperature=1.0, top_k=6, repeat_penalty=2.0, repeat_last_n=4)]:
        for seed in (1, 2, 3, 4, 5):
            g = TextGenerationConfig(1, seed=seed, **kw)
            got = LogitsSampler(seed).select_next_token(logits, ids, g)
            want = oracle.LogitsSampler(seed).select_next_token(host, ids, oracle.sampling(seed=seed, **kw))
            assert got == want, (kw, seed)


def test_sampler_skips_non_finite_logits():
    """Rows of wte made of infinities give +inf, -inf and NaN logits: sample_logits keeps the
    finite ones only (generation.rs:300-310), on the device path (top_k) as on the host path."""
    _, cfg, w, ids = small_cases()[1]
    ids = [t for t in ids if t not in (3, 4, 5)] or [1]
    wte = np.asarray(w.wte, np.float32).reshape(cfg.vocab_size, cfg.n_embd).copy()
    wte[3] = np.inf                                                   # mixed-sign hidden state: NaN
    wte[4] = 0.0
    wte[4, 0] = np.inf                                                # +inf or -inf
    wte[5] = 0.0
    wte[5, 0] = -np.inf
    w.wte = wte.reshape(-1)
    model = Gpt2Model.new(cfg, w)
    cache = model.new_kv_cache()
    logits = model.prefill(ids, cache)
    host = logits.to_host()
    assert not np.isfinite(host[[3, 4, 5]]).any() and np.isfinite(np.delete(host, [3, 4, 5])).all()
    for kw in [dict(temperature=1.0, top_k=5), dict(temperature=1.0, top_k=cfg.vocab_size - 3),
               dict(temperature=1.0, top_k=cfg.vocab_size - 1), dict(temperature=0.9, top_k=64, repeat_penalty=1.4),
               dict(temperature=1.0), dict(temperature=1.2, top_p=0.7)]:
        for seed in (5, 6, 7):
            g = TextGenerationConfig(1, seed=seed, **kw)
            got = LogitsSampler(seed).select_next_token(logits, ids, g)
            want = oracle.LogitsSampler(seed).select_next_token(host, ids, oracle.sampling(seed=seed, **kw))
            assert got == want and got not in (3, 4, 5), (kw, seed)


def test_sampled_stream_matches_oracle():
    _, cfg, w, ids = small_cases()[1]
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w)
    g = TextGenerationConfig(12, temperature=0.9, top_k=30, top_p=0.95, repeat_penalty=1.2, seed=7)
    toks, stats = model.stream_token_ids_with_stats(ids, g)
    want, st, _, _ = ref.stream_token_ids_with_stats(
        ids, 12, None, oracle.sampling(temperature=0.9, top_k=30, top_p=0.95, repeat_penalty=1.2, seed=7))
    assert toks == want and stats.generated_tokens == st.generated_tokens


def greedy_with_teacher_forcing(model, ref, ids, max_new, check_every=1):
    """Runs the oracle's greedy stream and replays its tokens through the HIP
    model, comparing logits at each step; returns (#steps, #argmax mismatches
    that the oracle's top-2 gap explains, #unexplained)."""
    want, st, rlogits, gaps = ref.stream_token_ids_with_stats(ids, max_new, None, want_logits=True)
    cache = model.new_kv_cache()
    logits = model.prefill(ids, cache)
    explained = unexplained = 0
    for step in range(st.generated_tokens):
        if step % check_every == 0:
            assert_logits_close(logits.to_host(), rlogits[step], what=f"step {step}")
        tok = model.select_next_token(logits)
        ref_tok = want[len(ids) + step]
        if tok != ref_tok:
            if gaps[step] <= 2 * (ABS_TOL + REL_TOL * abs(float(rlogits[step].max()))):
                explained += 1
            else:
                unexplained += 1
        if step + 1 < st.generated_tokens:
            logits = model.forward_one(ref_tok, cache)  # teacher-force the reference's token
    return st.generated_tokens, explained, unexplained, want


def test_config1_gpt2_small_greedy_decode_parity():
    """Benchmark configuration 1: 124M, 32 prompt ids, 128 greedy tokens with KV cache."""
    cfg = synth.Gpt2Config(**synth.GPT2_SMALL)
    w = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 1)
    ids = list(synth.token_ids(32, synth.TOKEN_SEED_BASE + 1, cfg.vocab_size))
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(8))
    steps, explained, unexplained, want = greedy_with_teacher_forcing(model, ref, ids, 128)
    assert steps == 128 and unexplained == 0
    # the fused on-device loop yields the same ids wherever no near-tie intervened
    cache = model.new_kv_cache()
    model.prefill(ids, cache)
    got, stats = model.decode_greedy(cache, 128)
    assert stats.generated_tokens == 128 and len(got) == 128
    if explained == 0:
        assert got == want[32:]
    assert cache.seq_len == 32 + 127  # the forward after the last token is skipped
    # A destroyed cache hands its block of tagged activation words back to a pool and the
    # next cache takes it over, old epochs and all: the result must not depend on that.
    for _ in range(3):
        del cache
        cache = model.new_kv_cache()
        model.prefill(ids, cache)
        again, _ = model.decode_greedy(cache, 128)
        assert again == got


def test_config2_gpt2_small_full_context_prefill_parity():
    """Benchmark configuration 2: 124M, one prompt of 1024 ids (the whole context) through the
    MFMA GEMM path and the full causal attention; final-position logits and the cache it
    leaves against the oracle's token-by-token prefill (rust.rs:906-927)."""
    cfg = synth.Gpt2Config(**synth.GPT2_SMALL)
    w = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 2)
    ids = list(synth.token_ids(1024, synth.TOKEN_SEED_BASE + 2, cfg.vocab_size))
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(16))
    cache, rcache = model.new_kv_cache(), ref.new_kv_cache()
    want = ref.prefill(ids, rcache)
    got = model.prefill(ids, cache)
    assert_logits_close(got.to_host(), want)
    assert model.select_next_token(got) == oracle.argmax_logits(want) or \
        np.diff(np.sort(want)[-2:])[0] <= 2 * (ABS_TOL + REL_TOL * abs(float(want.max())))
    assert cache.seq_len == 1024 == cache.max_seq_len
    for layer in (0, cfg.n_layer - 1):
        for which in (0, 1):
            np.testing.assert_allclose(cache.read_layer(layer, which), rcache.read_layer(layer, which),
                                       atol=2e-5, rtol=1e-4)
    # the context is used up (rust.rs:957-961)
    with pytest.raises(Gpt2Error, match="cache is full at seq_len 1024"):
        model.forward_one(1, cache)
    # prefill clears the cache first (rust.rs:913): a second prompt starts from position 0
    short = ids[:40]
    assert_logits_close(model.prefill(short, cache).to_host(), ref.prefill(short, rcache))
    assert cache.seq_len == 40


def test_config4_gpt2_xl_long_context_greedy_decode_parity():
    """Benchmark configuration 4, the headline workload: XL, cache prefilled with 896 ids, 128
    greedy tokens at positions 896..1022 (the context ends exactly there).  Logits of every
    step against the oracle with its tokens teacher-forced, then the fused on-device loop."""
    cfg = synth.Gpt2Config(**synth.GPT2_XL)
    w = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 4)
    ids = list(synth.token_ids(896, synth.TOKEN_SEED_BASE + 4, cfg.vocab_size))
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(16))
    assert "decode=persistent" in model.describe()
    steps, explained, unexplained, want = greedy_with_teacher_forcing(model, ref, ids, 128)
    assert steps == 128 and unexplained == 0
    assert len(want) == 1024  # stopped by the context limit, not short of it
    cache = model.new_kv_cache()
    model.prefill(ids, cache)
    got, stats = model.decode_greedy(cache, 128)
    assert stats.generated_tokens == 128 and len(got) == 128
    if explained == 0:
        assert got == want[896:]
    assert cache.seq_len == 896 + 127  # the forward after the last token is skipped


def sample_counts():
    import ctypes as C
    from puppygrad_amd import _lib
    dev, host = C.c_uint64(), C.c_uint64()
    _lib.load().pg_debug_sample_counts(C.byref(dev), C.byref(host))
    return dev.value, host.value


@pytest.mark.parametrize("vocab,ties", [(131, 0), (6011, 0), (50257, 0), (6011, 997)])
def test_sampling_without_top_k_is_drawn_on_the_device(vocab, ties):
    """Temperature and top-p sampling over the whole vocabulary (sample_logits,
    generation.rs:300-362) without the row of logits leaving the device: every draw equals the
    oracle's sampler on the same logits, and the library's counters show that no row was copied
    to the host.  With `ties`, wte rows repeat so that the stable order among equal logits
    decides which id a draw lands on."""
    cfg = synth.Gpt2Config(vocab_size=vocab, n_positions=32, n_embd=128, n_layer=1, n_head=2)
    w = synth.random_weights(cfg, 0x5EED0700 + vocab, std=0.05, perturb=True)
    if ties:
        wte = np.asarray(w.wte, np.float32).reshape(vocab, cfg.n_embd).copy()
        for i in range(vocab):
            wte[i] = wte[i % ties]
        wte[11] = np.inf
        wte[vocab - 5] = -np.inf
        w.wte = wte.reshape(-1)
    ids = [int(t) for t in synth.token_ids(9, 0x70C00700, min(vocab, 900)) if t != 11] or [1]
    model = Gpt2Model.new(cfg, w)
    cache = model.new_kv_cache()
    logits = model.prefill(ids, cache)
    host = logits.to_host()
    cases = [dict(temperature=1.0), dict(temperature=0.7), dict(temperature=2.5), dict(temperature=0.05),
             dict(temperature=1.0, top_p=0.9), dict(temperature=0.8, top_p=0.5), dict(temperature=1.3, top_p=0.05),
             dict(temperature=1.0, top_p=1.0), dict(temperature=1.0, top_p=0.999),
             dict(temperature=1.0, repeat_penalty=1.3), dict(temperature=0.9, top_p=0.8, repeat_penalty=0.7, repeat_last_n=4)]
    dev0, host0 = sample_counts()
    calls = 0
    for kw in cases:
        for seed in range(1, 13):
            g = TextGenerationConfig(1, seed=seed, **kw)
            sampler, ref_sampler = LogitsSampler(seed), oracle.LogitsSampler(seed)
            for draw in range(3):  # consecutive draws: the generator advances exactly as the oracle's
                got = sampler.select_next_token(logits, ids, g)
                want = ref_sampler.select_next_token(host, ids, oracle.sampling(seed=seed, **kw))
                assert got == want, (kw, seed, draw)
                calls += 1
    dev1, host1 = sample_counts()
    assert (dev1 - dev0) + (host1 - host0) == calls
    # (a draw within 1e-9 of a boundary would be repeated on the host; none is expected here)
    assert host1 - host0 <= 2 and dev1 - dev0 >= calls - 2


def test_sampling_over_equal_logits_falls_back_to_the_host():
    """A vocabulary whose logits are all equal: more candidates in one value bin than the device
    sorts, so the draw is repeated on the host, and still equals the oracle's."""
    cfg = synth.Gpt2Config(vocab_size=5003, n_positions=16, n_embd=64, n_layer=1, n_head=1)
    w = synth.random_weights(cfg, 0x5EED0710, perturb=True)
    wte = np.asarray(w.wte, np.float32).reshape(cfg.vocab_size, cfg.n_embd).copy()
    wte[:] = wte[0]
    w.wte = wte.reshape(-1)
    model = Gpt2Model.new(cfg, w)
    cache = model.new_kv_cache()
    logits = model.prefill([3, 4], cache)
    host = logits.to_host()
    assert len(np.unique(host)) == 1
    dev0, host0 = sample_counts()
    for seed in (1, 2, 3):
        got = LogitsSampler(seed).select_next_token(logits, [3, 4], TextGenerationConfig(1, seed=seed, temperature=1.0, top_p=0.7))
        want = oracle.LogitsSampler(seed).select_next_token(host, [3, 4], oracle.sampling(seed=seed, temperature=1.0, top_p=0.7))
        assert got == want
    dev1, host1 = sample_counts()
    assert host1 - host0 == 3 and dev1 == dev0


def test_sampled_stream_without_top_k_matches_oracle():
    _, cfg, w, ids = small_cases()[1]
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w)
    for kw in (dict(temperature=1.0), dict(temperature=0.8, top_p=0.9, repeat_penalty=1.2)):
        g = TextGenerationConfig(20, seed=11, **kw)
        toks, stats = model.stream_token_ids_with_stats(ids, g)
        want, st, _, _ = ref.stream_token_ids_with_stats(ids, 20, None, oracle.sampling(seed=11, **kw))
        assert toks == want and stats.generated_tokens == st.generated_tokens
