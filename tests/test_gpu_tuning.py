"""Models built with non-default tunables (what the autotune scan varies and
puppygrad-tune.json holds) stay parity-green, the tuning file of a model directory is picked
up, and a short scan runs end to end."""
import json

import numpy as np
import pytest

import oracle
from helpers import ABS_TOL, REL_TOL, assert_logits_close
from puppygrad_amd import Gpt2Config, Gpt2HipConfig, Gpt2Model, synth
from puppygrad_amd._lib import PG_STORE_BF16, PG_STORE_INT8
from puppygrad_amd.autotune import AutoTuneOptions, candidate_grid, load_gpt2_tuning, run_gpt2_autotune
from test_assets import write_model_dir

pytestmark = pytest.mark.gpu


def decode_against_oracle(model, ref, ids, forced=(7, 123, 42), n_greedy=6):
    cache, rcache = model.new_kv_cache(), ref.new_kv_cache()
    assert_logits_close(model.prefill(ids, cache).to_host(), ref.prefill(ids, rcache))
    rlog = None
    for tok in forced:
        rlog = ref.forward_one(tok, rcache)
        assert_logits_close(model.forward_one(tok, cache).to_host(), rlog)
    got, _ = model.decode_greedy(cache, n_greedy)
    want, clear = [], True
    for i in range(n_greedy):
        top = np.sort(rlog)[-2:]
        clear = clear and (top[1] - top[0]) > 2 * (ABS_TOL + REL_TOL * abs(float(top[1])))
        want.append(oracle.argmax_logits(rlog))
        if i + 1 < n_greedy:
            rlog = ref.forward_one(want[-1], rcache)
    assert len(got) == n_greedy
    if clear:
        assert got == want


@pytest.mark.parametrize("n_embd,n_head,n_prompt", [(768, 12, 100), (768, 12, 300), (768, 12, 900),
                                                    (1024, 16, 500), (1600, 25, 700)])
def test_fused_decode_with_256_key_attention_items(n_embd, n_head, n_prompt):
    """attn_item_keys = 256: half as many key splits per head (one up to 256 keys, four at 900
    where the default has eight), eight steps per key slot."""
    cfg = Gpt2Config(vocab_size=300, n_positions=1024, n_embd=n_embd, n_layer=1, n_head=n_head)
    w = synth.random_weights(cfg, 0x5EED0600 + n_head, perturb=True)
    ids = list(synth.token_ids(n_prompt, 0x70C00600 + n_prompt, cfg.vocab_size))
    model = Gpt2Model.new(cfg, w, Gpt2HipConfig(attn_item_keys=256))
    assert "decode=persistent" in model.describe() and "attn_item_keys=256" in model.describe()
    decode_against_oracle(model, oracle.Model(cfg, w, oracle.rust_config(8)), ids)


@pytest.mark.parametrize("storage", [PG_STORE_BF16, PG_STORE_INT8], ids=["bf16", "int8"])
def test_fused_decode_with_256_key_items_on_packed_rows(storage):
    cfg = Gpt2Config(vocab_size=300, n_positions=512, n_embd=768, n_layer=2, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0610, perturb=True)
    ids = list(synth.token_ids(400, 0x70C00610, cfg.vocab_size))
    model = Gpt2Model.new(cfg, w, Gpt2HipConfig(weight_storage=storage, attn_item_keys=256))
    assert "decode=persistent" in model.describe()
    if storage == PG_STORE_BF16:
        ref = oracle.Model(cfg, synth.bf16_rounded(w), oracle.rust_config(8))
    else:
        ref = oracle.Model(cfg, w, oracle.rust_config(8, quantized_weights=1))
    decode_against_oracle(model, ref, ids)


@pytest.mark.parametrize("blocks,items", [(1, 1), (16, 8), (2, 4)])
def test_per_operation_and_batched_paths_with_other_split_plans(blocks, items):
    """attn_blocks_per_cu moves the key-split count of the decode attention kernel,
    gemm_split_items_per_cu the K cuts of the tile GEMM: results stay the oracle's."""
    hip = Gpt2HipConfig(attn_blocks_per_cu=blocks, gemm_split_items_per_cu=items)
    cfg = Gpt2Config(vocab_size=211, n_positions=512, n_embd=128, n_layer=2, n_head=2)
    w = synth.random_weights(cfg, 0x5EED0620, perturb=True)
    ids = list(synth.token_ids(300, 0x70C00620, cfg.vocab_size))
    model, ref = Gpt2Model.new(cfg, w, hip), oracle.Model(cfg, w)
    assert f"attn_blocks_per_cu={blocks}" in model.describe()
    decode_against_oracle(model, ref, ids)
    # 124M's layer shapes at 512 tokens: the projections back to n_embd are cut along K
    cfg = Gpt2Config(vocab_size=97, n_positions=512, n_embd=768, n_layer=1, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0214, perturb=True)
    ids = list(synth.token_ids(512, 0x70C00214, 97))
    per_op = Gpt2Model.new(cfg, w, Gpt2HipConfig(decode_path=1, attn_blocks_per_cu=blocks,
                                                 gemm_split_items_per_cu=items))
    ref = oracle.Model(cfg, w, oracle.rust_config(8))
    cache, rcache = per_op.new_kv_cache(), ref.new_kv_cache()
    assert_logits_close(per_op.prefill(ids[:480], cache).to_host(), ref.prefill(ids[:480], rcache))
    for tok in (5, 6):
        assert_logits_close(per_op.forward_one(tok, cache).to_host(), ref.forward_one(tok, rcache))
    # a batch of five
    B, n = 5, 200
    bids = synth.token_ids(B * n, 0x70C00621, cfg.vocab_size).reshape(B, n)
    bc = per_op.new_kv_cache(B)
    got = per_op.prefill_batch(bids, bc).to_host()
    rcs = [ref.new_kv_cache() for _ in range(B)]
    want = np.stack([ref.prefill(bids[b], rcs[b]) for b in range(B)])
    assert_logits_close(got, want)
    nxt = np.argmax(want, axis=1).astype(np.uint32)
    got = per_op.forward_one_batch(nxt, bc).to_host()
    want = np.stack([ref.forward_one(int(nxt[b]), rcs[b]) for b in range(B)])
    assert_logits_close(got, want)


def test_planner_tunables_move_the_prompt_to_other_kernels_with_the_same_logits():
    """seq_gemm_min_tokens decides from which prompt length the GEMM prefill runs,
    gemm_b9_min_rows from which row count f32 products take the bf16 matrix cores: every
    setting gives the oracle's logits (the nine-product form is exact in its products)."""
    cfg = Gpt2Config(vocab_size=97, n_positions=512, n_embd=768, n_layer=1, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0650, perturb=True)
    ref = oracle.Model(cfg, w, oracle.rust_config(8))
    ids = [int(t) for t in synth.token_ids(512, 0x70C00650, 97)]
    want = {n: ref.prefill(ids[:n], ref.new_kv_cache()) for n in (6, 40, 512)}
    for kw in (dict(), dict(seq_gemm_min_tokens=2), dict(seq_gemm_min_tokens=48),
               dict(gemm_b9_min_rows=128), dict(gemm_b9_min_rows=0xffffffff)):
        model = Gpt2Model.new(cfg, w, Gpt2HipConfig(**kw))
        text = model.describe()
        assert f"seq_gemm_min_tokens={kw.get('seq_gemm_min_tokens', 4)}" in text
        assert f"gemm_b9_min_rows={min(kw.get('gemm_b9_min_rows', 1024), 0x7fffffff)}" in text
        for n, logits in want.items():
            cache = model.new_kv_cache()
            assert_logits_close(model.prefill(ids[:n], cache).to_host(), logits)
            assert cache.seq_len == n


def test_model_directory_tuning_file_is_read(tmp_path):
    cfg = Gpt2Config(vocab_size=300, n_positions=64, n_embd=768, n_layer=1, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0630, perturb=True)
    d = write_model_dir(tmp_path / "m", cfg, w)
    assert "attn_item_keys=128" in Gpt2Model.from_dir(d).describe()
    (d / "puppygrad-tune.json").write_text(json.dumps(
        {"model": "gpt2", "backend": "hip", "hip": {"attn_item_keys": 256, "attn_blocks_per_cu": 8}}))
    text = Gpt2Model.from_dir(d).describe()
    assert "attn_item_keys=256" in text and "attn_blocks_per_cu=8" in text and "gemm_split_items_per_cu=3" in text
    # what the caller sets wins over the file
    text = Gpt2Model.from_dir(d, Gpt2HipConfig(attn_item_keys=128)).describe()
    assert "attn_item_keys=128" in text and "attn_blocks_per_cu=8" in text
    tuned = load_gpt2_tuning(None, d)
    assert tuned.attn_item_keys == 256
    # a directory the reference's own scan has tuned (only a `rust` object in the file) loads with
    # this backend's defaults
    (d / "puppygrad-tune.json").write_text(json.dumps(
        {"model": "gpt2", "backend": "rust", "rust": {"parallel_attention_min_tokens": 64}}))
    text = Gpt2Model.from_dir(d).describe()
    assert "attn_item_keys=128" in text and "attn_blocks_per_cu=4" in text and "gemm_split_items_per_cu=3" in text


def test_autotune_scan_end_to_end(tmp_path):
    cfg = Gpt2Config(vocab_size=2003, n_positions=512, n_embd=768, n_layer=2, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0640, std=0.1, perturb=True)
    prompts = [[int(t) for t in synth.token_ids(200, 0x70C00640, cfg.vocab_size)]]
    candidates = candidate_grid(Gpt2HipConfig(), [128, 256], [4], [3])
    lines = []
    result, validation, score = run_gpt2_autotune(
        lambda hip: Gpt2Model.new(cfg, w, hip), prompts, 24, candidates,
        AutoTuneOptions(warmup_runs=1, measured_runs=2, max_trials=8), validation_runs=2,
        save_path=tmp_path / "puppygrad-tune.json", log=lines.append, eos_token_id=None)
    assert len(result.trials) == 2 and all(t.score > 0 for t in result.trials)
    assert result.best_score == max(t.score for t in result.trials) and score > 0
    assert validation.generated_tokens > 0 and validation.runs_per_prompt == 2
    assert any(line.startswith("autotune trial: attn_item_keys=256") for line in lines)
    saved = json.loads((tmp_path / "puppygrad-tune.json").read_text())
    assert saved["hip"]["attn_item_keys"] == result.best_config.attn_item_keys
    assert load_gpt2_tuning(tmp_path / "puppygrad-tune.json").attn_item_keys == result.best_config.attn_item_keys
    # the planner's knobs ranked by the whole generation's rate
    candidates = candidate_grid(Gpt2HipConfig(), [128], [4], [3], [0, 128], [4, 512])
    result, validation, score = run_gpt2_autotune(
        lambda hip: Gpt2Model.new(cfg, w, hip), prompts, 8, candidates,
        AutoTuneOptions(warmup_runs=1, measured_runs=2, max_trials=8), validation_runs=2,
        save_path=tmp_path / "planner.json", log=lines.append, eos_token_id=None, score_by="total")
    assert len(result.trials) == 4 and result.best_score == max(t.score for t in result.trials)
    assert all(t.score == t.measurement.total_tokens_per_second_median for t in result.trials)
    saved = json.loads((tmp_path / "planner.json").read_text())
    assert saved["score_name"] == "median_total_tokens_per_second"
    assert saved["hip"]["seq_gemm_min_tokens"] == result.best_config.seq_gemm_min_tokens
