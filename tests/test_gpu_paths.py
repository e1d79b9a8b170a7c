"""Device paths that only particular inputs reach: the EOS stop inside the fused greedy loop
and the rewind that follows it (src/models/gpt2/rust.rs:495-531: EOS is tested before the
push, never emitted, and no forward runs for it), the streamed form of that loop across
launch boundaries, batched decode deep into the context, one model shared by threads with
their own caches, and the restart of the exchange epochs."""
import ctypes as C
import threading

import numpy as np
import pytest

import oracle
from helpers import ABS_TOL, REL_TOL, assert_logits_close
from puppygrad_amd import (Gpt2Config, Gpt2Error, Gpt2HipConfig, Gpt2Model, TextGenerationConfig,
                           _lib, synth)
from puppygrad_amd._lib import PG_STORE_BF16

pytestmark = pytest.mark.gpu


def explained(tok, rlog):
    """The oracle picks `tok` too, or its top-2 gap is inside the logit tolerance."""
    if tok == oracle.argmax_logits(rlog):
        return True
    top = float(np.max(rlog))
    return top - float(rlog[tok]) <= 2 * (ABS_TOL + REL_TOL * abs(top))


class Replay:
    """The oracle fed with the GPU's own tokens: cache state after prompt + any prefix."""

    def __init__(self, ref, ids):
        self.ref, self.ids = ref, list(ids)
        self.cache = ref.new_kv_cache()
        self.logits = ref.prefill(self.ids, self.cache)
        self.fed = []

    def feed(self, tok):
        self.logits = self.ref.forward_one(int(tok), self.cache)
        self.fed.append(int(tok))

    def rewind_to(self, toks):
        """State after prompt + toks (a prefix of what was fed is kept, the rest re-run)."""
        toks = [int(t) for t in toks]
        keep = 0
        while keep < min(len(toks), len(self.fed)) and toks[keep] == self.fed[keep]:
            keep += 1
        self.cache.seq_len = len(self.ids) + keep
        self.fed = self.fed[:keep]
        if keep == 0:
            self.logits = self.ref.prefill(self.ids, self.cache)
        for t in toks[keep:]:
            self.feed(t)


EOS_CASES = [
    # name, config, weight std, prompt length, tokens to generate
    ("persistent768", dict(vocab_size=2003, n_positions=256, n_embd=768, n_layer=2, n_head=12), 0.1, 20, 150),
    ("persistent1600", dict(vocab_size=2003, n_positions=128, n_embd=1600, n_layer=2, n_head=25), 0.08, 30, 70),
    ("per_op128", dict(vocab_size=257, n_positions=96, n_embd=128, n_layer=2, n_head=2), 0.2, 17, 40),
]


@pytest.mark.parametrize("case", EOS_CASES, ids=lambda c: c[0])
def test_eos_stops_the_greedy_loop_and_rewinds_the_cache(case):
    name, kw, std, n_prompt, n_new = case
    cfg = Gpt2Config(**kw)
    w = synth.random_weights(cfg, 0x5EED0400 + n_prompt, std=std, perturb=True)
    ids = [int(t) for t in synth.token_ids(n_prompt, 0x70C00400 + n_prompt, cfg.vocab_size)]
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(8))
    assert ("decode=persistent" in model.describe()) == name.startswith("persistent")

    # the unconstrained greedy run of the fused loop, checked token by token against the oracle
    cache = model.new_kv_cache()
    model.prefill(ids, cache)
    base, st = model.decode_greedy(cache, n_new)
    assert len(base) == n_new == st.generated_tokens and cache.seq_len == n_prompt + n_new - 1
    rep = Replay(ref, ids)
    for i, tok in enumerate(base):
        assert explained(tok, rep.logits), f"token {i} of the free run"
        if i + 1 < n_new:
            rep.feed(tok)
    assert len(set(base)) > n_new // 4  # a varied stream: late tokens are first occurrences

    picks = sorted({0, 1, 2, n_new // 2, 63, 64, 65, 128, 129, n_new - 2, n_new - 1} & set(range(n_new)))
    firsts = set()
    for k in picks:
        eos = base[k]
        j = base.index(eos)  # the run stops where this id first shows up
        firsts.add(j)
        # fused loop on a prefilled cache
        model.prefill(ids, cache)
        got, st = model.decode_greedy(cache, n_new, eos=eos)
        assert got == base[:j] and st.generated_tokens == j, (k, j)
        assert cache.seq_len == n_prompt + j  # one forward per emitted token, none for EOS
        # the cache really is in that state: the next forward matches the oracle's
        rep.rewind_to(base[:j])
        probe = (eos + 1) % cfg.vocab_size
        if cache.seq_len < cfg.n_positions:
            want = ref.forward_one(probe, rep.cache)
            rep.cache.seq_len -= 1
            assert_logits_close(model.forward_one(probe, cache).to_host(), want, what=f"after eos at {j}")
        # the streamed loop (the entry point the reference's CLI calls)
        seen = []
        toks, stats = model.stream_token_ids_with_stats(
            ids, TextGenerationConfig(n_new, eos_token_id=eos), seen.append)
        assert toks == ids + base[:j] and seen == base[:j], (k, j)
        assert stats.generated_tokens == j and stats.prompt_tokens == n_prompt
        assert (stats.first_token_time is None) == (j == 0)
    assert len(firsts) >= 4  # stops at the first token, in the middle and late were all seen

    # no EOS in sight: the stream is the free run, delivered in order
    seen = []
    toks, stats = model.stream_token_ids_with_stats(ids, TextGenerationConfig(n_new), seen.append)
    assert toks == ids + base and seen == base and stats.generated_tokens == n_new
    # the oracle's own loop agrees wherever no near-tie intervened
    want, rst, rlogits, gaps = ref.stream_token_ids_with_stats(ids, n_new, None, want_logits=True)
    if (gaps > 2 * (ABS_TOL + REL_TOL * np.abs(rlogits).max(axis=1))).all():
        assert toks == want
    # the context limit ends the stream (rust.rs:496-498)
    room = cfg.n_positions - n_prompt
    toks, stats = model.stream_token_ids_with_stats(ids, TextGenerationConfig(room + 50))
    assert len(toks) == cfg.n_positions and stats.generated_tokens == room
    assert toks[:n_prompt + n_new] == ids + base


def test_stream_callback_failure_ends_the_generation():
    name, kw, std, n_prompt, n_new = EOS_CASES[0]
    cfg = Gpt2Config(**kw)
    w = synth.random_weights(cfg, 0x5EED0400 + n_prompt, std=std, perturb=True)
    ids = [int(t) for t in synth.token_ids(n_prompt, 0x70C00400 + n_prompt, cfg.vocab_size)]
    model = Gpt2Model.new(cfg, w)
    seen = []

    def on_token(tok):
        seen.append(tok)
        if len(seen) == 5:
            raise RuntimeError("stop here")

    with pytest.raises(RuntimeError, match="stop here"):
        model.stream_token_ids_with_stats(ids, TextGenerationConfig(100), on_token)
    assert len(seen) == 5
    # the model is as usable as before
    again = []
    toks, _ = model.stream_token_ids_with_stats(ids, TextGenerationConfig(8), again.append)
    assert again == seen[:5] + again[5:] and toks == ids + again

    # a callback that calls the model while its own generation runs is refused, not deadlocked
    cache = model.new_kv_cache()
    model.prefill(ids, cache)
    errors = []

    def reenter(tok):
        if not errors:
            try:
                model.forward_one(tok, cache)
                errors.append(None)
            except Gpt2Error as e:
                errors.append(str(e))

    toks2, _ = model.stream_token_ids_with_stats(ids, TextGenerationConfig(8), reenter)
    assert toks2 == toks
    assert errors and (errors[0] is None or "must not call the model" in errors[0])


def test_threads_share_a_model_with_their_own_caches():
    """One model, several threads, one cache each (the boundary's threading contract): fused
    decodes, streamed generations and GEMM prefills interleave and every thread gets the ids
    a single thread gets."""
    cfg = Gpt2Config(vocab_size=2003, n_positions=256, n_embd=768, n_layer=2, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0410, std=0.1, perturb=True)
    model = Gpt2Model.new(cfg, w)
    assert "decode=persistent" in model.describe()
    prompts = [[int(t) for t in synth.token_ids(n, 0x70C00410 + n, cfg.vocab_size)] for n in (5, 21, 40, 90)]
    n_new = 48

    def run(ids):
        cache = model.new_kv_cache()
        model.prefill(ids, cache)
        toks, _ = model.decode_greedy(cache, n_new)
        streamed, _ = model.stream_token_ids_with_stats(ids, TextGenerationConfig(n_new))
        return toks, streamed[len(ids):]

    want = [run(p) for p in prompts]
    for toks, streamed in want:
        assert toks == streamed
    results = {}
    failures = []

    def worker(i):
        try:
            for r in range(4):
                results[(i, r)] = run(prompts[i])
        except Exception as e:  # surfaced below
            failures.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(prompts))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not failures, failures
    for (i, r), got in results.items():
        assert got == want[i], (i, r)

    # the same with the per-operation launches of a shape the fused kernel does not take
    cfg2 = Gpt2Config(vocab_size=257, n_positions=96, n_embd=128, n_layer=2, n_head=2)
    small = Gpt2Model.new(cfg2, synth.random_weights(cfg2, 0x5EED0411, std=0.2, perturb=True))
    p2 = [[int(t) for t in synth.token_ids(n, 0x70C00420 + n, cfg2.vocab_size)] for n in (3, 19, 33)]

    def run2(ids):
        cache = small.new_kv_cache()
        small.prefill(ids, cache)
        return small.decode_greedy(cache, 30)[0]

    want2 = [run2(p) for p in p2]
    got2 = {}

    def worker2(i):
        for r in range(4):
            got2[(i, r)] = run2(p2[i])

    threads = [threading.Thread(target=worker2, args=(i,)) for i in range(len(p2))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads)
    assert len(got2) == 12 and all(v == want2[i] for (i, _), v in got2.items())


def test_exchange_epochs_restart_near_their_limit():
    """The tagged words of the fused decode kernel carry a 32-bit epoch.  A cache moved to just
    below the limit (test hook) runs launches at the highest epochs, then one that clears the
    words and starts from 1 again; the ids never change."""
    cfg = Gpt2Config(vocab_size=2003, n_positions=256, n_embd=768, n_layer=2, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0410, std=0.1, perturb=True)
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(8))
    ids = [int(t) for t in synth.token_ids(30, 0x70C00430, cfg.vocab_size)]
    lib = _lib.load()
    cache = model.new_kv_cache()
    model.prefill(ids, cache)
    base, _ = model.decode_greedy(cache, 10)
    rep = Replay(ref, ids)
    for tok in base:
        assert explained(tok, rep.logits)
        rep.feed(tok)
    limit = 0xE0000000
    assert 0 < lib.pg_kv_cache_debug_epoch(cache._h) < 10_000
    assert lib.pg_kv_cache_debug_set_epoch(cache._h, limit - 300) == 0
    assert lib.pg_kv_cache_debug_set_epoch(cache._h, 5) != 0  # never backwards
    seen = []
    for _ in range(4):
        model.prefill(ids, cache)
        got, _ = model.decode_greedy(cache, 10)
        assert got == base
        seen.append(lib.pg_kv_cache_debug_epoch(cache._h))
    assert seen[0] > limit - 300 and min(seen) < 10_000, seen  # ran high, then restarted
    # single forwards right after the restart
    model.prefill(ids, cache)
    rep.rewind_to([])
    for tok in base[:3]:
        assert_logits_close(model.forward_one(tok, cache).to_host(), ref.forward_one(tok, rep.cache))


DEEP_CASES = [
    # the attention shapes of the batched benchmark configurations: heads x batch = 256 (355M,
    # batch 16) and 800 (XL, batch 32, bf16 weights), one layer so that the oracle stays cheap
    ("h16_b16_f32", dict(vocab_size=257, n_positions=1024, n_embd=1024, n_layer=1, n_head=16), 16, 0),
    ("h25_b32_bf16", dict(vocab_size=257, n_positions=1024, n_embd=1600, n_layer=1, n_head=25), 32, PG_STORE_BF16),
]


@pytest.mark.parametrize("case", DEEP_CASES, ids=lambda c: c[0])
def test_batched_decode_deep_in_the_context(case):
    """Batched steps at cache lengths around 130, 520, 1000 and at the very end of the context:
    the split count and the chunk depth of the batched attention kernel depend on the key
    count.  Logits of the first and last sequence and the K/V rows the steps append, against
    the oracle."""
    name, kw, B, storage = case
    cfg = Gpt2Config(**kw)
    w = synth.random_weights(cfg, 0x5EED0440 + B, std=0.05, perturb=True)
    if storage == PG_STORE_BF16:
        w = synth.bf16_rounded(w)
    model = Gpt2Model.new(cfg, w, Gpt2HipConfig(weight_storage=storage))
    ref = oracle.Model(cfg, w, oracle.rust_config(8))
    all_ids = synth.token_ids(B * 1024, 0x70C00440 + B, cfg.vocab_size).reshape(B, 1024)
    check = [0, B - 1]
    cache = model.new_kv_cache(B)
    rc = {b: ref.new_kv_cache() for b in check}
    done = {b: 0 for b in check}  # prompt tokens the oracle's cache of sequence b holds
    for n, steps in ((130, 3), (520, 3), (1000, 3), (1020, 4)):
        ids = np.ascontiguousarray(all_ids[:, :n])
        logits = model.prefill_batch(ids, cache).to_host()
        want = {}
        for b in check:
            # the oracle extends its cache token by token (prompts share their prefix)
            rc[b].seq_len = done[b]
            for t in all_ids[b, done[b]:n]:
                want[b] = ref.forward_one(int(t), rc[b])
            done[b] = n
            assert_logits_close(logits[b], want[b], what=f"{name} prefill {n} seq {b}")
        nxt = np.argmax(logits, axis=1).astype(np.uint32)
        for step in range(steps):
            for b in check:
                nxt[b] = int(np.argmax(want[b]))
            logits = model.forward_one_batch(nxt, cache).to_host()
            for b in check:
                want[b] = ref.forward_one(int(nxt[b]), rc[b])
                assert_logits_close(logits[b], want[b], what=f"{name} {n}+{step} seq {b}")
            nxt = np.argmax(logits, axis=1).astype(np.uint32)
        assert cache.seq_len == n + steps
        for b in check:
            for which in (0, 1):
                np.testing.assert_allclose(cache.read_layer(0, which, b)[:, :n + steps],
                                           rc[b].read_layer(0, which)[:, :n + steps], atol=2e-5, rtol=1e-4)
    assert cache.seq_len == 1024
    with pytest.raises(Gpt2Error, match="cache is full at seq_len 1024"):
        model.forward_one_batch(nxt, cache)


def test_config3_gpt2_medium_batch16_to_the_end():
    """Benchmark configuration 3 in full: 355M, batch 16, 128-token prompts, 256 greedy tokens
    (255 steps, the caches grow to 383 keys).  All sequences run on the GPU; sequences 0 and 15
    are teacher-forced with the oracle's tokens and compared every 16th step and at the last."""
    cfg = Gpt2Config(**synth.GPT2_MEDIUM)
    B, n, steps = 16, 128, 255
    w = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 3)
    ids = synth.token_ids(B * n, synth.TOKEN_SEED_BASE + 3, cfg.vocab_size).reshape(B, n)
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(16))
    cache = model.new_kv_cache(B)
    logits = model.prefill_batch(ids, cache)
    check = [0, 15]
    rc = {b: ref.new_kv_cache() for b in check}
    want = {b: ref.prefill(ids[b], rc[b]) for b in check}
    nxt = logits.argmax()
    for step in range(steps):
        for b in check:
            nxt[b] = int(np.argmax(want[b]))
        logits = model.forward_one_batch(nxt, cache)
        for b in check:
            want[b] = ref.forward_one(int(nxt[b]), rc[b])
        if step % 16 == 0 or step == steps - 1:
            host = logits.to_host()
            for b in check:
                assert_logits_close(host[b], want[b], what=f"step {step} seq {b}")
        nxt = logits.argmax()
    assert cache.seq_len == n + steps == 383
