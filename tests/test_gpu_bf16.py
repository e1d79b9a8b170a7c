"""bf16 weight storage (benchmark configuration 5): the token embedding and the block matrices
are kept as bf16 in HBM, accumulation / LayerNorm / softmax / KV cache stay f32.  The
oracle runs on the same bf16-rounded weights widened to f32, so both sides multiply
identical values and the f32 tolerance applies; the 2e-2 relative bound the config
states is checked against un-rounded weights as well."""
import numpy as np
import pytest

import oracle
from helpers import assert_logits_close
from puppygrad_amd import Gpt2Config, Gpt2Error, Gpt2HipConfig, Gpt2Model, synth
from puppygrad_amd._lib import PG_DECODE_PERSISTENT, PG_STORE_BF16

pytestmark = pytest.mark.gpu

BF16 = Gpt2HipConfig(weight_storage=PG_STORE_BF16)


def test_bf16_rounding_is_nearest_even():
    """Values chosen on rounding boundaries: ties go to the even mantissa."""
    bits = np.array([0x3F800000, 0x3F808000, 0x3F818000, 0x3F808001, 0x3F807FFF, 0xBF808000,
                     0x00000001, 0x7F7FFFFF], dtype=np.uint32)
    want = np.array([0x3F80, 0x3F80, 0x3F82, 0x3F81, 0x3F80, 0xBF80, 0x0000, 0x7F80],
                    dtype=np.uint32) << 16
    np.testing.assert_array_equal(synth.round_bf16(bits.view(np.float32)).view(np.uint32), want)


@pytest.mark.parametrize("n_embd,n_head,n_prompt", [(128, 2, 21), (192, 3, 5), (100, 5, 18), (128, 2, 36)])
def test_bf16_storage_matches_oracle_on_rounded_weights(n_embd, n_head, n_prompt):
    cfg = Gpt2Config(vocab_size=263, n_positions=40, n_embd=n_embd, n_layer=2, n_head=n_head)
    w = synth.random_weights(cfg, 0x5EED0500 + n_embd, perturb=True)
    wr = synth.bf16_rounded(w)
    ids = synth.token_ids(n_prompt, 0x70C00500, cfg.vocab_size)
    model, ref = Gpt2Model.new(cfg, w, BF16), oracle.Model(cfg, wr)
    assert "weights=bf16" in model.describe()
    cache, rc = model.new_kv_cache(), ref.new_kv_cache()
    got, want = model.prefill(ids, cache).to_host(), ref.prefill(ids, rc)
    assert_logits_close(got, want)
    for _ in range(4):
        tok = int(np.argmax(want))
        got, want = model.forward_one(tok, cache).to_host(), ref.forward_one(tok, rc)
        assert_logits_close(got, want)
    assert_logits_close(model.forward(ids).logits, ref.forward(ids))
    # against the un-rounded f32 weights: the config's 2e-2 relative bound
    full = oracle.Model(cfg, w).forward(ids)
    scale = np.abs(full).max()
    assert np.abs(model.forward(ids).logits - full).max() <= 2e-2 * scale


@pytest.mark.parametrize("n_embd,n_head,n_prompt", [(832, 13, 400), (768, 12, 512)])
def test_bf16_long_prompts_on_the_bf16_matrix_cores(n_embd, n_head, n_prompt):
    """Prompts long enough that c_attn and c_fc run as 128 x 128 tiles on the bf16 matrix cores,
    the f32 inputs cut into three bf16 parts (exact products, f32 sums): a ragged last row tile
    (400 = 3 x 128 + 16), widths that are no multiple of the tile (2496, 3328) and ones that
    are, against the oracle on the rounded weights at the f32 tolerance."""
    cfg = Gpt2Config(vocab_size=300, n_positions=512, n_embd=n_embd, n_layer=1, n_head=n_head)
    w = synth.random_weights(cfg, 0x5EED0520 + n_head, perturb=True)
    ids = synth.token_ids(n_prompt, 0x70C00520, cfg.vocab_size)
    model = Gpt2Model.new(cfg, w, BF16)
    ref = oracle.Model(cfg, synth.bf16_rounded(w), oracle.rust_config(8))
    cache, rc = model.new_kv_cache(), ref.new_kv_cache()
    want = ref.prefill(ids, rc)
    assert_logits_close(model.prefill(ids, cache).to_host(), want)
    full = model.forward(ids).logits
    assert_logits_close(full, ref.forward(ids))
    if n_prompt < cfg.n_positions:
        tok = int(np.argmax(want))
        assert_logits_close(model.forward_one(tok, cache).to_host(), ref.forward_one(tok, rc))


def test_bf16_batched_steps():
    cfg = Gpt2Config(vocab_size=257, n_positions=48, n_embd=128, n_layer=2, n_head=2)
    B, n = 6, 20
    w = synth.random_weights(cfg, 0x5EED0501, perturb=True)
    ids = synth.token_ids(B * n, 0x70C00501, cfg.vocab_size).reshape(B, n)
    model, ref = Gpt2Model.new(cfg, w, BF16), oracle.Model(cfg, synth.bf16_rounded(w))
    cache = model.new_kv_cache(B)
    got = model.prefill_batch(ids, cache).to_host()
    rcs = [ref.new_kv_cache() for _ in range(B)]
    want = np.stack([ref.prefill(ids[b], rcs[b]) for b in range(B)])
    assert_logits_close(got, want)
    nxt = np.argmax(want, axis=1).astype(np.uint32)
    for _ in range(3):
        got = model.forward_one_batch(nxt, cache).to_host()
        want = np.stack([ref.forward_one(int(nxt[b]), rcs[b]) for b in range(B)])
        assert_logits_close(got, want)
        nxt = np.argmax(want, axis=1).astype(np.uint32)


def test_bf16_options_are_validated():
    cfg = Gpt2Config(vocab_size=257, n_positions=48, n_embd=128, n_layer=1, n_head=2)
    w = synth.random_weights(cfg, 3)
    with pytest.raises(Gpt2Error, match="decode_path=persistent needs head_dim 64"):
        Gpt2Model.new(cfg, w, Gpt2HipConfig(weight_storage=PG_STORE_BF16,
                                            decode_path=PG_DECODE_PERSISTENT))
    with pytest.raises(Gpt2Error, match="weight_storage must be f32, bf16 or int8"):
        Gpt2Model.new(cfg, w, Gpt2HipConfig(weight_storage=7))


@pytest.mark.parametrize("n_embd,n_head,n_prompt", [(768, 12, 20), (1024, 16, 150), (1280, 20, 70), (1600, 25, 40)])
def test_bf16_persistent_decode_matches_oracle(n_embd, n_head, n_prompt):
    """The persistent decode kernel on bf16 rows (8 weights per 16-byte chunk, bf16 embedding
    table): single forwards and a multi-token launch against the oracle on the rounded
    weights, and against the per-op path."""
    cfg = Gpt2Config(vocab_size=300, n_positions=256, n_embd=n_embd, n_layer=2, n_head=n_head)
    w = synth.random_weights(cfg, 0x5EED0510 + n_head, perturb=True)
    ids = list(synth.token_ids(n_prompt, 0x70C00510, cfg.vocab_size))
    model, ref = Gpt2Model.new(cfg, w, BF16), oracle.Model(cfg, synth.bf16_rounded(w), oracle.rust_config(8))
    assert "weights=bf16" in model.describe() and "decode=persistent" in model.describe()
    per_op = Gpt2Model.new(cfg, w, Gpt2HipConfig(weight_storage=PG_STORE_BF16, decode_path=1))
    assert "decode=kernels" in per_op.describe()
    cache, pcache, rcache = model.new_kv_cache(), per_op.new_kv_cache(), ref.new_kv_cache()
    assert_logits_close(model.prefill(ids, cache).to_host(), ref.prefill(ids, rcache))
    per_op.prefill(ids, pcache)
    rlog = None
    for tok in (7, 123, 42):
        rlog = ref.forward_one(tok, rcache)
        got = model.forward_one(tok, cache).to_host()
        assert_logits_close(got, rlog)
        assert_logits_close(got, per_op.forward_one(tok, pcache).to_host(), abs_tol=2e-5, rel_tol=1e-4)
    got, _ = model.decode_greedy(cache, 6)  # five forwards in one launch
    want, clear = [], True
    for i in range(6):
        top = np.sort(rlog)[-2:]
        clear = clear and (top[1] - top[0]) > 2 * (1e-4 + 1e-3 * abs(float(top[1])))
        want.append(oracle.argmax_logits(rlog))
        if i < 5:
            rlog = ref.forward_one(want[-1], rcache)
    assert len(got) == 6
    if clear:
        assert got == want


def test_config5_gpt2_xl_bf16_batch32_subsample():
    """Benchmark configuration 5 shape (XL, bf16 weights, batch 32, 512-token prompts): all 32
    sequences run on the GPU; sequence 0 and 31 are checked against the oracle (on the
    rounded weights) for the prompt and 3 teacher-forced steps."""
    cfg = Gpt2Config(**synth.GPT2_XL)
    B, n, steps = 32, 512, 3
    w = synth.bf16_rounded(synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 5))
    ids = synth.token_ids(B * n, synth.TOKEN_SEED_BASE + 5, cfg.vocab_size).reshape(B, n)
    model, ref = Gpt2Model.new(cfg, w, BF16), oracle.Model(cfg, w, oracle.rust_config(16))
    cache = model.new_kv_cache(B)
    logits = model.prefill_batch(ids, cache).to_host()
    check = [0, 31]
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


def test_config5_full_depth_sequence0_to_the_context_limit():
    """Benchmark configuration 5 at its full depth on the full model (XL, 48 layers, bf16 weights,
    batch 32, 512-token prompts, 511 steps to position 1022): sequence 0 is teacher-forced with
    the oracle's greedy tokens through every step, the other 31 sequences follow their own argmax.
    Its logits are compared with the oracle's (on the rounded weights, f32 tolerance) at the first
    step, at about 1000 keys and at the last two positions, so that what 48 layers of the
    three-part bf16 products do to the error at nearly full context is pinned, not only its
    start."""
    cfg = Gpt2Config(**synth.GPT2_XL)
    B, n = 32, 512
    steps = cfg.n_positions - 1 - n  # forwards at positions 512..1022
    w = synth.bf16_rounded(synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 5))
    ids = synth.token_ids(B * n, synth.TOKEN_SEED_BASE + 5, cfg.vocab_size).reshape(B, n)
    model, ref = Gpt2Model.new(cfg, w, BF16), oracle.Model(cfg, w, oracle.rust_config(16))
    cache = model.new_kv_cache(B)
    logits = model.prefill_batch(ids, cache).to_host()
    rc = ref.new_kv_cache()
    want = ref.prefill(ids[0], rc)
    assert_logits_close(logits[0], want, what="prefill seq 0")
    checked = {0, 255, 487, 488, steps - 2, steps - 1}  # positions 512, 767, 999, 1000, 1021, 1022
    worst = 0.0
    for step in range(steps):
        nxt = np.argmax(logits, axis=1).astype(np.uint32)
        nxt[0] = int(np.argmax(want))
        logits = model.forward_one_batch(nxt, cache).to_host()
        want = ref.forward_one(int(nxt[0]), rc)
        if step in checked:
            assert_logits_close(logits[0], want, what=f"step {step} (position {n + step}) seq 0")
            worst = max(worst, float(np.abs(logits[0] - want).max()))
    assert cache.seq_len == cfg.n_positions - 1 and rc.seq_len == cfg.n_positions - 1
    print(f"config 5 full depth: max |logit error| of sequence 0 at the checked steps {worst:.2e}")
