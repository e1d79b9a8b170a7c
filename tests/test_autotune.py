"""The autotune scan in the reference's shape (src/models/autotune.rs:1-85, the GPT-2 target in
src/main.rs:2587-2958): selection rule, trial limit, the measurement arithmetic, the candidate
grid, and the saved file as the library reads it back.  No GPU needed."""
import ctypes as C
import json

import pytest

from puppygrad_amd import Gpt2Error, Gpt2HipConfig, Gpt2Model, _lib, synth
from puppygrad_amd.autotune import (AutoTuneOptions, Gpt2AutoTuneMeasurement, autotune, candidate_grid,
                                    load_gpt2_tuning, save_gpt2_tuning, summarize_runs)
from puppygrad_amd.gpt2 import GenerationStats


class FakeTarget:
    def __init__(self, scores):
        self.scores = scores
        self.seen = []

    def candidate_configs(self):
        return list(range(len(self.scores)))

    def evaluate_config(self, config, options):
        self.seen.append(config)
        return {"tps": self.scores[config], "runs": options.measured_runs}

    def score(self, measurement):
        return measurement["tps"]


def test_autotune_keeps_the_first_strictly_best_candidate():
    target = FakeTarget([3.0, 7.5, 7.5, 1.0])
    result = autotune(target, AutoTuneOptions(measured_runs=2))
    assert result.best_config == 1 and result.best_score == 7.5  # the tie at index 2 does not win
    assert [t.config for t in result.trials] == [0, 1, 2, 3] and target.seen == [0, 1, 2, 3]
    assert [t.score for t in result.trials] == [3.0, 7.5, 7.5, 1.0]
    assert result.trials[0].measurement == {"tps": 3.0, "runs": 2}


def test_autotune_evaluates_at_most_max_trials_candidates():
    target = FakeTarget([1.0, 2.0, 9.0])
    result = autotune(target, AutoTuneOptions(max_trials=2))
    assert target.seen == [0, 1] and result.best_config == 1
    with pytest.raises(ValueError, match="at least one candidate"):
        autotune(FakeTarget([]), AutoTuneOptions())


def test_measurement_arithmetic():
    # two runs: 10 tokens in 0.5 s and 30 tokens in 1.0 s (decode); prefill 0.1 s and 0.3 s
    stats = [GenerationStats(4, 10, 0.1, 0.5, 0.01), GenerationStats(6, 30, 0.3, 1.0, 0.02)]
    m = summarize_runs(0.25, prompt_count=1, runs_per_prompt=2, stats=stats)
    assert m.load_ms == 250.0 and m.generated_tokens == 40 and m.prompt_count == 1 and m.runs_per_prompt == 2
    assert m.decode_tokens_per_second == pytest.approx(40 / 1.5)       # of the summed times
    assert m.decode_tokens_per_second_median == pytest.approx(25.0)    # rates 20 and 30
    assert m.decode_tokens_per_second_p25 == pytest.approx(22.5)
    assert m.decode_tokens_per_second_p95 == pytest.approx(29.5)
    assert m.decode_tokens_per_second_stddev == pytest.approx(5.0)     # population sigma
    assert m.total_tokens_per_second == pytest.approx(50 / 1.9)
    assert m.total_tokens_per_second_median == pytest.approx((14 / 0.6 + 36 / 1.3) / 2)
    assert m.prefill_ms == pytest.approx(200.0) and m.decode_ms == pytest.approx(750.0)
    assert m.total_generation_ms == pytest.approx(950.0)
    empty = summarize_runs(0.0, 0, 0, [])
    assert empty == Gpt2AutoTuneMeasurement()


def test_candidate_grid_is_the_cross_product_in_order():
    grid = candidate_grid(Gpt2HipConfig(weight_storage=2), [128, 256], [2, 4], [3])
    assert [(g.attn_item_keys, g.attn_blocks_per_cu, g.gemm_split_items_per_cu) for g in grid] == \
        [(128, 2, 3), (128, 4, 3), (256, 2, 3), (256, 4, 3)]
    assert all(g.weight_storage == 2 for g in grid)
    grid = candidate_grid(Gpt2HipConfig(), [128], [4], [3], [512, 2048], [2, 16])
    assert [(g.gemm_b9_min_rows, g.seq_gemm_min_tokens) for g in grid] == [(512, 2), (512, 16), (2048, 2), (2048, 16)]
    with pytest.raises(ValueError, match="no candidates"):
        candidate_grid(Gpt2HipConfig(), [], [4], [3])


def test_saved_tuning_round_trip(tmp_path):
    best = Gpt2HipConfig(attn_item_keys=256, attn_blocks_per_cu=8, gemm_split_items_per_cu=2)
    meas = Gpt2AutoTuneMeasurement(prompt_count=2, decode_tokens_per_second_median=2200.5)
    path = tmp_path / "m" / "puppygrad-tune.json"
    save_gpt2_tuning(path, best, 2190.0, 2200.5, meas, 64, AutoTuneOptions(1, 5, None), "medium")
    saved = json.loads(path.read_text())
    assert list(saved) == ["model", "backend", "score_name", "score", "search_score", "max_new_tokens",
                           "warmup_runs", "measured_runs", "prompt_count", "hip", "measurement"]
    assert saved["backend"] == "hip" and saved["score_name"] == "median_decode_tokens_per_second"
    assert saved["score"] == 2200.5 and saved["search_score"] == 2190.0 and saved["prompt_count"] == 2
    assert saved["hip"] == {"attn_item_keys": 256, "attn_blocks_per_cu": 8, "gemm_split_items_per_cu": 2,
                            "gemm_b9_min_rows": 0, "seq_gemm_min_tokens": 0}
    assert saved["measurement"]["decode_tokens_per_second_median"] == 2200.5
    # the library's reader: the default file of a model directory, and an explicit file
    got = load_gpt2_tuning(None, tmp_path / "m")
    assert (got.attn_item_keys, got.attn_blocks_per_cu, got.gemm_split_items_per_cu) == (256, 8, 2)
    got = load_gpt2_tuning(path, None, Gpt2HipConfig(attn_blocks_per_cu=6, weight_storage=1))
    assert (got.attn_item_keys, got.attn_blocks_per_cu, got.weight_storage) == (256, 6, 1)  # explicit wins
    # the planner's knobs and the score they were ranked by
    best = Gpt2HipConfig(gemm_b9_min_rows=512, seq_gemm_min_tokens=8)
    save_gpt2_tuning(tmp_path / "p.json", best, 1.0, 2.0, meas, 8, AutoTuneOptions(1, 5, None), "small", "total")
    saved = json.loads((tmp_path / "p.json").read_text())
    assert saved["score_name"] == "median_total_tokens_per_second"
    got = load_gpt2_tuning(tmp_path / "p.json", None)
    assert (got.gemm_b9_min_rows, got.seq_gemm_min_tokens, got.attn_item_keys) == (512, 8, 0)
    assert load_gpt2_tuning(None, tmp_path) is None  # no default file: nothing to load
    with pytest.raises(FileNotFoundError, match="does not exist"):
        load_gpt2_tuning(tmp_path / "nope.json", None)


def test_malformed_tuning_files_are_asset_errors(tmp_path):
    lib = _lib.load()
    opts = _lib.pg_hip_options()
    found = C.c_int32(5)
    assert lib.pg_hip_load_tuning(str(tmp_path / "absent.json").encode(), C.byref(opts), C.byref(found)) == 0
    assert found.value == 0
    for text, why in [("{", "failed to parse tuning file"), ("[1]", "expected an object of per-backend tunings"),
                      ('{"hip": 3}', "invalid type for field `hip`"),
                      ('{"hip": {"attn_item_keys": "x"}}', "invalid type for field `attn_item_keys`"),
                      ('{"hip": {"attn_blocks_per_cu": -1}}', "invalid type for field `attn_blocks_per_cu`"),
                      ('{"hip": {"gemm_split_items_per_cu": 2.5}}', "expected u32")]:
        p = tmp_path / "t.json"
        p.write_text(text)
        assert lib.pg_hip_load_tuning(str(p).encode(), C.byref(opts), C.byref(found)) == _lib.PG_ASSET
        assert why in lib.pg_last_error_message().decode()
    # a file the reference's own `autotune gpt2` wrote (SavedGpt2Tuning, main.rs:2611-2623: a `rust`
    # object and no `hip`) is no tuning for this backend, and no error
    for text in ['{"rust": {"parallel_attention_min_tokens": 64}}', '{"hip": null}', "{}"]:
        p.write_text(text)
        opts = _lib.pg_hip_options()
        found = C.c_int32(5)
        assert lib.pg_hip_load_tuning(str(p).encode(), C.byref(opts), C.byref(found)) == 0
        assert found.value == 0
        assert (opts.attn_item_keys, opts.attn_blocks_per_cu, opts.gemm_split_items_per_cu) == (0, 0, 0)
    p.write_text('{"hip": {"attn_item_keys": 256, "unknown": 1, "attn_blocks_per_cu": null}}')
    opts = _lib.pg_hip_options()
    assert lib.pg_hip_load_tuning(str(p).encode(), C.byref(opts), C.byref(found)) == 0 and found.value == 1
    assert (opts.attn_item_keys, opts.attn_blocks_per_cu, opts.gemm_split_items_per_cu) == (256, 0, 0)


def test_tunables_are_validated_before_any_device_work():
    cfg = synth.tiny_config()
    w = synth.tiny_weights(cfg)
    for kw, msg in [(dict(attn_item_keys=100), "attn_item_keys must be 0 \\(default\\), 128 or 256"),
                    (dict(attn_blocks_per_cu=65), "attn_blocks_per_cu must be at most 64"),
                    (dict(gemm_split_items_per_cu=17), "gemm_split_items_per_cu must be at most 16"),
                    (dict(seq_gemm_min_tokens=65537), "seq_gemm_min_tokens must be at most 65536")]:
        with pytest.raises(Gpt2Error, match=msg) as e:
            Gpt2Model.new(cfg, w, Gpt2HipConfig(**kw))
        assert e.value.kind == "InvalidConfig"
