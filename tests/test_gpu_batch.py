"""Batched decode (the batched benchmark configurations: 355M batch 16, XL bf16 batch 32): every sequence of a batch must
match the oracle run on that sequence alone."""
import numpy as np
import pytest

import oracle
from helpers import ABS_TOL, REL_TOL, assert_logits_close
from puppygrad_amd import Gpt2Config, Gpt2Error, Gpt2HipConfig, Gpt2Model, synth

pytestmark = pytest.mark.gpu


def batch_case(seed, B, n, cfg):
    w = synth.random_weights(cfg, 0x5EED0300 + seed, perturb=True)
    ids = synth.token_ids(B * n, 0x70C00300 + seed, cfg.vocab_size).reshape(B, n)
    return w, ids


@pytest.mark.parametrize("prefill_path", [0, 1], ids=["gemm_prefill", "token_prefill"])
@pytest.mark.parametrize("B,n", [(3, 21), (16, 17), (2, 5), (17, 6), (20, 9), (32, 7), (40, 5)])
def test_batched_steps_match_oracle(B, n, prefill_path):
    cfg = Gpt2Config(vocab_size=257, n_positions=48, n_embd=128, n_layer=2, n_head=2)
    w, ids = batch_case(B * 100 + n, B, n, cfg)
    model = Gpt2Model.new(cfg, w, Gpt2HipConfig(prefill_path=prefill_path))
    ref = oracle.Model(cfg, w)
    cache = model.new_kv_cache(B)
    assert cache.batch == B
    got = model.prefill_batch(ids, cache).to_host()
    rcaches = [ref.new_kv_cache() for _ in range(B)]
    want = np.stack([ref.prefill(ids[b], rcaches[b]) for b in range(B)])
    assert_logits_close(got, want)
    assert cache.seq_len == n
    nxt = np.argmax(want, axis=1).astype(np.uint32)
    for _ in range(3):
        got = model.forward_one_batch(nxt, cache).to_host()
        want = np.stack([ref.forward_one(int(nxt[b]), rcaches[b]) for b in range(B)])
        assert_logits_close(got, want)
        nxt = np.argmax(want, axis=1).astype(np.uint32)
    for b in (0, B - 1):  # per-sequence K/V panels
        np.testing.assert_allclose(cache.read_layer(1, 0, b)[:, :cache.seq_len],
                                   rcaches[b].read_layer(1, 0)[:, :cache.seq_len], atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("storage", [0, 1], ids=["f32", "bf16"])
def test_small_batch_of_a_wide_model_matches_oracle(storage):
    """n_embd above 1024: even a batch of 4 runs its projections on the 32-row MFMA kernel,
    with the activations between them in that kernel's packed layout."""
    cfg = Gpt2Config(vocab_size=211, n_positions=40, n_embd=1088, n_layer=2, n_head=17)
    B, n = 4, 11
    w, ids = batch_case(31, B, n, cfg)
    if storage:
        for blk in w.blocks:
            for f in ("c_attn_w", "c_proj_w", "c_fc_w", "c_proj_mlp_w"):
                setattr(blk, f, synth.round_bf16(getattr(blk, f)))
        w.wte = synth.round_bf16(w.wte)
    model = Gpt2Model.new(cfg, w, Gpt2HipConfig(weight_storage=storage))
    ref = oracle.Model(cfg, w, oracle.rust_config(8))
    cache = model.new_kv_cache(B)
    got = model.prefill_batch(ids, cache).to_host()
    rcaches = [ref.new_kv_cache() for _ in range(B)]
    want = np.stack([ref.prefill(ids[b], rcaches[b]) for b in range(B)])
    assert_logits_close(got, want)
    nxt = np.argmax(want, axis=1).astype(np.uint32)
    for step in range(3):
        got = model.forward_one_batch(nxt, cache).to_host()
        want = np.stack([ref.forward_one(int(nxt[b]), rcaches[b]) for b in range(B)])
        assert_logits_close(got, want, what=f"step {step}")
        nxt = np.argmax(want, axis=1).astype(np.uint32)


def test_batched_greedy_decode_matches_oracle_tokens():
    cfg = Gpt2Config(vocab_size=257, n_positions=64, n_embd=128, n_layer=2, n_head=2)
    B, n, steps = 5, 19, 12
    w, ids = batch_case(7, B, n, cfg)
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w)
    cache = model.new_kv_cache(B)
    model.prefill_batch(ids, cache)
    got, stats = model.decode_greedy_batch(cache, steps)
    assert got.shape == (steps, B) and stats.generated_tokens == steps
    assert cache.seq_len == n + steps - 1  # no forward after the last selected token
    for b in range(B):
        want, st, logits, gaps = ref.stream_token_ids_with_stats(ids[b], steps, None, want_logits=True)
        if (gaps > 2 * (ABS_TOL + REL_TOL * np.abs(logits).max())).all():
            assert [int(t) for t in got[:, b]] == want[n:]


def test_batch_argument_errors():
    cfg = Gpt2Config(vocab_size=257, n_positions=48, n_embd=128, n_layer=1, n_head=2)
    w, ids = batch_case(9, 2, 4, cfg)
    model = Gpt2Model.new(cfg, w)
    cache = model.new_kv_cache(2)
    with pytest.raises(Gpt2Error, match="needs a cache of batch 1"):
        model.prefill(ids[0], cache)
    with pytest.raises(Gpt2Error, match="one id per sequence"):
        model.forward_one_batch([1], cache)
    bad = ids.copy()
    bad[1, 2] = 257
    with pytest.raises(Gpt2Error, match="token id 257 at index 2 exceeds vocab_size 257"):
        model.prefill_batch(bad, cache)
    with pytest.raises(Gpt2Error, match="cache batch must be > 0"):
        model.new_kv_cache(0)


def test_config3_gpt2_medium_batch16_subsample():
    """Benchmark configuration 3 (355M, batch 16, 128-token prompts): all 16 sequences run on the
    GPU; sequences 0, 7 and 15 are checked against the oracle for the prompt and the
    first 6 greedy steps (teacher-forced with the oracle's tokens)."""
    cfg = Gpt2Config(**synth.GPT2_MEDIUM)
    B, n, steps = 16, 128, 6
    w = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 3)
    ids = synth.token_ids(B * n, synth.TOKEN_SEED_BASE + 3, cfg.vocab_size).reshape(B, n)
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(16))
    cache = model.new_kv_cache(B)
    logits = model.prefill_batch(ids, cache).to_host()
    check = [0, 7, 15]
    rc = {b: ref.new_kv_cache() for b in check}
    want = {b: ref.prefill(ids[b], rc[b]) for b in check}
    for b in check:
        assert_logits_close(logits[b], want[b], what=f"prefill seq {b}")
    nxt = np.argmax(logits, axis=1).astype(np.uint32)
    for b in check:
        nxt[b] = int(np.argmax(want[b]))
    for step in range(steps):
        logits = model.forward_one_batch(nxt, cache).to_host()
        for b in check:
            want[b] = ref.forward_one(int(nxt[b]), rc[b])
            assert_logits_close(logits[b], want[b], what=f"step {step} seq {b}")
        nxt = np.argmax(logits, axis=1).astype(np.uint32)
        for b in check:
            nxt[b] = int(np.argmax(want[b]))
