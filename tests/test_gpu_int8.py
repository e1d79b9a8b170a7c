"""int8 weight storage (the reference's `quantized_weights` option): the library quantises
the block matrices and the lm_head copy of wte on the device and multiplies with
(float)q * scale (the matrix-vector kernels per weight, the matrix-core kernels per row sum);
the oracle's quantised path (pinned in test_oracle_int8.py) is the reference.  Both sides use
identical quantised values and scales, so the f32 tolerance applies."""
import numpy as np
import pytest

import oracle
from helpers import ABS_TOL, REL_TOL, assert_logits_close, small_cases
from puppygrad_amd import Gpt2Config, Gpt2Error, Gpt2HipConfig, Gpt2Model, synth
from puppygrad_amd._lib import PG_STORE_INT8

pytestmark = pytest.mark.gpu

INT8 = Gpt2HipConfig(weight_storage=PG_STORE_INT8)


def qref(cfg, w, threads=1):
    return oracle.Model(cfg, w, oracle.rust_config(threads, quantized_weights=1))


def test_quantized_rust_forward_returns_finite_logits():
    # rust.rs:1996-2013 on this backend
    cfg = synth.tiny_config()
    w = synth.tiny_weights(cfg)
    out = Gpt2Model.new(cfg, w, INT8).forward([1, 2, 3]).logits
    assert out.shape == (3, cfg.vocab_size) and np.isfinite(out).all()
    assert_logits_close(out, qref(cfg, w).forward([1, 2, 3]))


@pytest.mark.parametrize("case", small_cases(), ids=lambda c: c[0])
def test_int8_storage_matches_the_quantised_oracle(case):
    """tiny (K = 4, scalar loads), c128 (16-byte int8 loads, GEMM prefill), odd (n_embd 36:
    no 16-byte path, token-by-token prefill)."""
    name, cfg, w, ids = case
    model, ref = Gpt2Model.new(cfg, w, INT8), qref(cfg, w)
    assert "weights=int8" in model.describe()
    cache, rc = model.new_kv_cache(), ref.new_kv_cache()
    got, want = model.prefill(ids, cache).to_host(), ref.prefill(ids, rc)
    assert_logits_close(got, want, what=f"{name} prefill")
    for step in range(min(4, cfg.n_positions - len(ids))):
        tok = int(np.argmax(want))
        got, want = model.forward_one(tok, cache).to_host(), ref.forward_one(tok, rc)
        assert_logits_close(got, want, what=f"{name} step {step}")
    assert_logits_close(model.forward(ids).logits, ref.forward(ids), what=f"{name} forward")
    # the quantisation is really in effect: the f32 model differs
    assert np.abs(model.forward(ids).logits - oracle.Model(cfg, w).forward(ids)).max() > 1e-4


@pytest.mark.parametrize("n_embd,n_head,n_prompt", [(832, 13, 400), (768, 12, 512), (1024, 16, 100),
                                                    (1024, 16, 512)])
def test_int8_long_prompts_on_the_bf16_matrix_cores(n_embd, n_head, n_prompt):
    """Prompts of more than 64 tokens whose projections have a dozen 128 x 128 tiles or more run
    on the bf16 matrix cores (int8 values are bf16 numbers; the inputs are cut into three bf16
    parts; the row's scale multiplies the row's sum): tiles cut along K, whole tiles for c_fc of
    the last case (128 tiles), a ragged last row tile and widths that are no multiple of the
    tile, against the quantised oracle at the f32 tolerance."""
    cfg = Gpt2Config(vocab_size=300, n_positions=512, n_embd=n_embd, n_layer=1, n_head=n_head)
    w = synth.random_weights(cfg, 0x5EED0620 + n_head, perturb=True)
    ids = synth.token_ids(n_prompt, 0x70C00620, cfg.vocab_size)
    model, ref = Gpt2Model.new(cfg, w, INT8), qref(cfg, w, threads=8)
    cache, rc = model.new_kv_cache(), ref.new_kv_cache()
    want = ref.prefill(ids, rc)
    assert_logits_close(model.prefill(ids, cache).to_host(), want)
    assert_logits_close(model.forward(ids).logits, ref.forward(ids))
    if n_prompt < cfg.n_positions:
        tok = int(np.argmax(want))
        assert_logits_close(model.forward_one(tok, cache).to_host(), ref.forward_one(tok, rc))


def test_int8_extreme_rows():
    """A zero row (scale 1), a row with one huge entry and rows of tiny values keep the
    quantiser's edge cases on the device equal to the oracle's."""
    cfg = Gpt2Config(vocab_size=97, n_positions=24, n_embd=64, n_layer=1, n_head=1)
    w = synth.random_weights(cfg, 0x5EED0601, perturb=True)
    b = w.blocks[0]
    m = np.asarray(b.c_fc_w, np.float32).reshape(64, 256).copy()  # [in,out]: a column is a row of [out,in]
    m[:, 0] = 0.0
    m[:, 1] *= 1e-20
    m[5, 2] = 1000.0
    m[:, 3] = np.where(np.arange(64) % 2 == 0, 0.5, -1.0) * 127  # exact halves after scaling
    b.c_fc_w = m.reshape(-1)
    wte = np.asarray(w.wte, np.float32).reshape(97, 64).copy()
    wte[7] = 0.0
    w.wte = wte.reshape(-1)
    ids = synth.token_ids(9, 0x70C00601, 97)
    ids[3] = 7
    model, ref = Gpt2Model.new(cfg, w, INT8), qref(cfg, w)
    assert_logits_close(model.forward(ids).logits, ref.forward(ids))


def test_int8_batched_steps():
    cfg = Gpt2Config(vocab_size=257, n_positions=48, n_embd=128, n_layer=2, n_head=2)
    B, n = 5, 18
    w = synth.random_weights(cfg, 0x5EED0602, perturb=True)
    ids = synth.token_ids(B * n, 0x70C00602, cfg.vocab_size).reshape(B, n)
    model, ref = Gpt2Model.new(cfg, w, INT8), qref(cfg, w)
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


def test_int8_greedy_decode_matches_oracle_tokens():
    cfg = Gpt2Config(vocab_size=257, n_positions=64, n_embd=128, n_layer=2, n_head=2)
    w = synth.random_weights(cfg, 0x5EED0603, perturb=True)
    ids = [int(t) for t in synth.token_ids(13, 0x70C00603, 257)]
    model, ref = Gpt2Model.new(cfg, w, INT8), qref(cfg, w)
    want, _, logits, gaps = ref.stream_token_ids_with_stats(ids, 16, None, want_logits=True)
    got = model.generate_greedy_cached(ids, 16)
    if (gaps > 2 * (ABS_TOL + REL_TOL * np.abs(logits).max())).all():
        assert got == want


def test_int8_gpt2_small_decode_steps():
    """GPT-2 124M shapes (768 -> 2304 / 768 / 3072, 3072 -> 768, lm_head over 50257 rows):
    a 24-token prompt through the GEMM prefill and 3 decode steps against the oracle."""
    cfg = Gpt2Config(**synth.GPT2_SMALL)
    w = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 1)
    ids = synth.token_ids(24, synth.TOKEN_SEED_BASE + 1, cfg.vocab_size)
    model, ref = Gpt2Model.new(cfg, w, INT8), qref(cfg, w, threads=8)
    cache, rc = model.new_kv_cache(), ref.new_kv_cache()
    got, want = model.prefill(ids, cache).to_host(), ref.prefill(ids, rc)
    assert_logits_close(got, want, what="prefill")
    for step in range(3):
        tok = int(np.argmax(want))
        got, want = model.forward_one(tok, cache).to_host(), ref.forward_one(tok, rc)
        assert_logits_close(got, want, what=f"step {step}")


@pytest.mark.parametrize("n_embd,n_head,n_prompt", [(768, 12, 20), (1024, 16, 150), (1280, 20, 70), (1600, 25, 40)])
def test_int8_persistent_decode_matches_oracle(n_embd, n_head, n_prompt):
    """The persistent decode kernel on int8 rows (16 weights per 16-byte chunk; the XL rows
    are not whole runs of 64 chunks): single forwards and a multi-token launch against the
    quantised oracle, and against the per-op path on the same device weights."""
    cfg = Gpt2Config(vocab_size=300, n_positions=256, n_embd=n_embd, n_layer=2, n_head=n_head)
    w = synth.random_weights(cfg, 0x5EED0610 + n_head, perturb=True)
    ids = list(synth.token_ids(n_prompt, 0x70C00610, cfg.vocab_size))
    model, ref = Gpt2Model.new(cfg, w, INT8), qref(cfg, w, threads=8)
    assert "weights=int8" in model.describe() and "decode=persistent" in model.describe()
    per_op = Gpt2Model.new(cfg, w, Gpt2HipConfig(weight_storage=PG_STORE_INT8, decode_path=1))
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
        clear = clear and (top[1] - top[0]) > 2 * (ABS_TOL + REL_TOL * abs(float(top[1])))
        want.append(oracle.argmax_logits(rlog))
        if i < 5:
            rlog = ref.forward_one(want[-1], rcache)
    assert len(got) == 6
    if clear:
        assert got == want


def test_int8_options_are_validated():
    cfg = synth.tiny_config()
    w = synth.tiny_weights(cfg)
    with pytest.raises(Gpt2Error, match="weight_storage must be f32, bf16 or int8"):
        Gpt2Model.new(cfg, w, Gpt2HipConfig(weight_storage=3))
