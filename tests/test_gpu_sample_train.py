"""Sampled and penalised generation on the persistent decode path: the reference's loop
(src/models/gpt2/rust.rs:495-531: select, EOS test before the push, on_token, forward_one unless
it was the last token) runs as a train of launches whose selections (sample_logits,
src/models/generation.rs:281-362) keep the generator's state, the id history and the next
forward's id on the device.  Every id must be the one the oracle's sampler picks on the logits
of the device's own forwards, whether the device decided the draw or handed it to the host."""
import ctypes as C

import numpy as np
import pytest

import oracle
from puppygrad_amd import Gpt2Config, Gpt2Error, Gpt2Model, TextGenerationConfig, _lib, synth

pytestmark = pytest.mark.gpu


def sample_counts():
    dev, host = C.c_uint64(), C.c_uint64()
    _lib.load().pg_debug_sample_counts(C.byref(dev), C.byref(host))
    return dev.value, host.value


class step_by_step:
    """Streams select one pg_logits_sample call at a time while this is entered."""

    def __enter__(self):
        self.prev = _lib.load().pg_debug_sample_train(0)

    def __exit__(self, *exc):
        _lib.load().pg_debug_sample_train(self.prev)


def replay(model, ids, g):
    """The reference's loop with the oracle's sampler on the logits of the library's own
    single-step forwards: (all ids, generated count)."""
    cache = model.new_kv_cache()
    logits = model.prefill(ids, cache)
    sampler = oracle.LogitsSampler(g.seed)
    cfg = oracle.sampling(temperature=g.temperature, top_p=g.top_p, top_k=g.top_k, seed=g.seed,
                          repeat_penalty=g.repeat_penalty, repeat_last_n=g.repeat_last_n)
    out = list(ids)
    generated = 0
    for _ in range(g.max_new_tokens):
        if len(out) >= model.config.n_positions:
            break
        tok = sampler.select_next_token(logits.to_host(), out, cfg)
        if g.eos_token_id is not None and tok == g.eos_token_id:
            break
        out.append(tok)
        generated += 1
        if generated < g.max_new_tokens and len(out) < model.config.n_positions:
            logits = model.forward_one(tok, cache)
    return out, generated


def small_persistent(width=768, vocab=2003, positions=256, seed=0x5EED0900, std=0.1, layers=2):
    cfg = Gpt2Config(vocab_size=vocab, n_positions=positions, n_embd=width, n_layer=layers,
                     n_head=width // 64)
    w = synth.random_weights(cfg, seed + width, std=std, perturb=True)
    return cfg, w


SAMPLINGS = [
    dict(temperature=1.0),
    dict(temperature=0.8, top_p=0.9),
    dict(temperature=0.8, top_k=40),
    dict(temperature=1.1, top_k=7, top_p=0.6, repeat_penalty=1.3),
    dict(temperature=0.9, top_p=0.8, repeat_penalty=0.7, repeat_last_n=4),
    dict(temperature=0.0, repeat_penalty=1.5, repeat_last_n=16),
    dict(temperature=0.0, top_k=5, repeat_penalty=1.2),
    dict(temperature=1.0, top_k=4096),
    dict(temperature=0.7, top_k=200, top_p=0.95, repeat_penalty=1.1),
    dict(temperature=1.4, top_k=128),
    dict(temperature=0.6, top_k=1),
]


@pytest.mark.parametrize("width", [768, 1600])
def test_sampled_streams_in_trains_pick_the_oracles_ids(width):
    cfg, w = small_persistent(width, positions=256 if width == 768 else 128)
    model = Gpt2Model.new(cfg, w)
    assert "decode=persistent" in model.describe()
    ids = [int(t) for t in synth.token_ids(19, 0x70C00900, cfg.vocab_size)]
    n_new = 75 if width == 768 else 40  # more than two trains / more than one
    for i, kw in enumerate(SAMPLINGS if width == 768 else SAMPLINGS[1:5]):
        g = TextGenerationConfig(n_new, seed=100 + i, **kw)
        want, want_generated = replay(model, ids, g)
        dev0, host0 = sample_counts()
        seen = []
        got, stats = model.stream_token_ids_with_stats(ids, g, seen.append)
        dev1, host1 = sample_counts()
        assert got == want, kw
        assert stats.generated_tokens == want_generated == n_new and seen == got[len(ids):]
        assert stats.gpu_decode_time > 0.0
        # decided on the device (a draw within 1e-9 of a boundary would go to the host)
        assert dev1 - dev0 >= n_new - 2 and host1 - host0 <= 2, kw
        with step_by_step():
            again, _ = model.stream_token_ids_with_stats(ids, g)
        assert again == want, kw


def test_trains_of_a_model_with_an_odd_number_of_layers():
    """With an odd number of layers a forward leaves the other set of exchange words armed than
    the next one starts from, so every step of a train arms for its forward; with an even number
    only the first does.  Both must give the oracle's ids, also right after a greedy launch."""
    cfg, w = small_persistent(768, layers=3, seed=0x5EED0930)
    model = Gpt2Model.new(cfg, w)
    assert "decode=persistent" in model.describe()
    ids = [int(t) for t in synth.token_ids(11, 0x70C00930, cfg.vocab_size)]
    for i, kw in enumerate((SAMPLINGS[2], SAMPLINGS[1], SAMPLINGS[5])):
        g = TextGenerationConfig(40, seed=300 + i, **kw)
        want, want_generated = replay(model, ids, g)
        # a greedy stream in between: its launch ends with the exchange words in the other state
        model.stream_token_ids_with_stats(ids, TextGenerationConfig(5, seed=1, temperature=0.0))
        got, stats = model.stream_token_ids_with_stats(ids, g)
        assert got == want and stats.generated_tokens == want_generated == 40, kw


def test_train_stops_at_eos_at_the_context_limit_and_for_the_callback():
    cfg, w = small_persistent(768)
    model = Gpt2Model.new(cfg, w)
    ids = [int(t) for t in synth.token_ids(30, 0x70C00901, cfg.vocab_size)]
    kw = dict(temperature=0.9, top_k=50, repeat_penalty=1.1)
    free, _ = model.stream_token_ids_with_stats(ids, TextGenerationConfig(70, seed=5, **kw))
    assert len(free) == 100
    # an id of the free run as EOS: in the first train, on a train's last slot, in a later train
    for at in (3, 31, 32, 50):
        eos = free[30 + at]
        first = free[30:].index(eos)
        g = TextGenerationConfig(70, seed=5, eos_token_id=eos, **kw)
        got, stats = model.stream_token_ids_with_stats(ids, g)
        assert got == free[:30 + first] and stats.generated_tokens == first
        assert (got, first) == replay(model, ids, g)
    # the context ends the run: 256 positions, 250 of them the prompt
    long_ids = [int(t) for t in synth.token_ids(250, 0x70C00902, cfg.vocab_size)]
    g = TextGenerationConfig(40, seed=6, **kw)
    got, stats = model.stream_token_ids_with_stats(long_ids, g)
    assert len(got) == 256 and stats.generated_tokens == 6
    assert (got, 6) == replay(model, long_ids, g)
    # one token only: no forward at all
    g = TextGenerationConfig(1, seed=7, **kw)
    got, stats = model.stream_token_ids_with_stats(ids, g)
    assert (got, 1) == replay(model, ids, g) and stats.generated_tokens == 1
    # a callback that raises stops the generation with the library's error
    calls = []

    def stop_at_5(tok):
        calls.append(tok)
        if len(calls) == 5:
            raise RuntimeError("enough")

    with pytest.raises(RuntimeError, match="enough"):
        model.stream_token_ids_with_stats(ids, TextGenerationConfig(70, seed=5, **kw), stop_at_5)
    assert calls == free[30:35]
    # and the model still generates afterwards
    again, _ = model.stream_token_ids_with_stats(ids, TextGenerationConfig(70, seed=5, **kw))
    assert again == free


def test_draws_the_device_leaves_undecided_are_made_by_the_host_inside_a_stream():
    """Every logit equal: more candidates in one value bin than the device sorts, so every
    selection halts its train and is repeated by the host from the logits left in place."""
    cfg, w = small_persistent(768, vocab=5003, positions=64, seed=0x5EED0910)
    wte = np.asarray(w.wte, np.float32).reshape(cfg.vocab_size, cfg.n_embd).copy()
    wte[:] = wte[0]
    w.wte = wte.reshape(-1)
    model = Gpt2Model.new(cfg, w)
    assert "decode=persistent" in model.describe()
    ids = [3, 4, 5]
    g = TextGenerationConfig(9, seed=21, temperature=1.0, top_p=0.7)
    want, n = replay(model, ids, g)
    dev0, host0 = sample_counts()
    got, stats = model.stream_token_ids_with_stats(ids, g)
    dev1, host1 = sample_counts()
    assert got == want and stats.generated_tokens == n == 9
    assert host1 - host0 == 9
    # with top_k the 40 (300) lowest ids are the candidates: the stable order among equal values
    for k in (40, 300):
        g = TextGenerationConfig(9, seed=22, temperature=1.0, top_k=k)
        want, n = replay(model, ids, g)
        got, stats = model.stream_token_ids_with_stats(ids, g)
        assert got == want and max(got[3:]) < k


def test_a_row_without_a_finite_logit_ends_the_stream_with_the_references_error():
    cfg, w = small_persistent(768, vocab=1009, positions=64, seed=0x5EED0920)
    wte = np.asarray(w.wte, np.float32).reshape(cfg.vocab_size, cfg.n_embd).copy()
    wte[:] = np.inf
    w.wte = wte.reshape(-1)
    model = Gpt2Model.new(cfg, w)
    for kw in (dict(temperature=1.0), dict(temperature=1.0, top_k=10)):
        with pytest.raises(Gpt2Error, match="cannot sample from empty or non-finite logits"):
            model.stream_token_ids_with_stats([1, 2, 3], TextGenerationConfig(5, seed=3, **kw))
