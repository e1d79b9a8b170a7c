"""Experiment rows in the reference's schema (run_gpt2_experiment, src/main.rs:3440-3541;
Gpt2ExperimentRow, src/main.rs:3356-3402): the row arithmetic and the CSV form on the host,
and the profiled generation they are filled from on the GPU."""
import math

import numpy as np
import pytest

import oracle
from puppygrad_amd import GenerationStats, Gpt2Model, Gpt2OperationProfile, TextGenerationConfig, synth
from puppygrad_amd import experiment as ex

# The header line print_gpt2_experiment_csv writes (src/main.rs:3934-3936).
REFERENCE_CSV_HEADER = (
    "backend,prompt_index,prompt,threads,dense_parallel_threshold,qkv_chunk_size,"
    "attention_projection_chunk_size,mlp_fc_chunk_size,mlp_projection_chunk_size,logits_chunk_size,"
    "attention_head_parallel_threshold,quantized_weights,max_new_tokens,runs,prompt_tokens,"
    "generated_tokens,load_ms,tokenize_ms,prefill_ms,time_to_first_token_ms,decode_ms,"
    "total_generation_ms,decode_ms_min,decode_ms_median,decode_ms_p95,decode_ms_max,decode_ms_stddev,"
    "total_generation_ms_min,total_generation_ms_median,total_generation_ms_p95,"
    "total_generation_ms_max,total_generation_ms_stddev,prefill_tokens_per_second,"
    "decode_tokens_per_second,total_tokens_per_second,profile_tokenization_ms,profile_layer_norm_ms,"
    "profile_qkv_projection_ms,profile_attention_ms,profile_attention_projection_ms,"
    "profile_mlp_fc_projection_ms,profile_mlp_projection_ms,profile_final_logits_ms,"
    "profile_decoding_ms")


def test_csv_columns_are_the_reference_header():
    assert ",".join(ex.CSV_COLUMNS) == REFERENCE_CSV_HEADER
    assert ex.format_csv([]).strip() == REFERENCE_CSV_HEADER


def test_percentile_interpolates_between_ranks():
    v = [1.0, 2.0, 3.0, 4.0]
    assert ex.percentile(v, 0.5) == 2.5          # rank 1.5
    assert ex.percentile(v, 0.25) == 1.75        # rank 0.75
    assert ex.percentile(v, 0.95) == pytest.approx(3.85)  # rank 2.85
    assert ex.percentile(v, 0.0) == 1.0 and ex.percentile(v, 1.0) == 4.0
    assert ex.percentile(v, 7.0) == 4.0 and ex.percentile(v, -1.0) == 1.0  # clamped
    assert ex.percentile([], 0.5) == 0.0
    assert ex.percentile([5.0], 0.95) == 5.0


def test_value_distribution_uses_population_stddev():
    d = ex.value_distribution([4.0, 1.0, 3.0, 2.0])  # unsorted on purpose
    assert (d.min, d.median, d.max) == (1.0, 2.5, 4.0)
    assert d.stddev == pytest.approx(math.sqrt(1.25))  # divides by n, not n - 1
    z = ex.value_distribution([])
    assert (z.min, z.p25, z.median, z.p95, z.max, z.stddev) == (0.0,) * 6


def _stats(generated, prefill, decode, first=0.01, prompt=7):
    return GenerationStats(prompt, generated, prefill, decode, first, 0.0)


def test_average_row_takes_rates_from_mean_times():
    stats = [_stats(4, 0.010, 0.020), _stats(4, 0.030, 0.060)]
    prof = [Gpt2OperationProfile(qkv_projection=0.001, attention=0.002, final_logits=0.004),
            Gpt2OperationProfile(qkv_projection=0.003, attention=0.002, final_logits=0.000)]
    r = ex.average_row("hip", False, 0, "p", 4, 1.5, stats, prof)
    assert r.runs == 2 and r.prompt_tokens == 7 and r.generated_tokens == 4.0
    assert r.load_ms == pytest.approx(1500.0)
    assert r.prefill_ms == pytest.approx(20.0) and r.decode_ms == pytest.approx(40.0)
    assert r.total_generation_ms == pytest.approx(60.0)
    assert r.prefill_tokens_per_second == pytest.approx(7 / 0.020)
    assert r.decode_tokens_per_second == pytest.approx(4 / 0.040)   # generated / decode time
    assert r.total_tokens_per_second == pytest.approx(11 / 0.060)
    assert (r.decode_ms_min, r.decode_ms_max) == (pytest.approx(20.0), pytest.approx(60.0))
    assert r.decode_ms_median == pytest.approx(40.0) and r.decode_ms_stddev == pytest.approx(20.0)
    assert r.total_generation_ms_p95 == pytest.approx(30.0 + 0.95 * 60.0)
    assert r.profile_qkv_projection_ms == pytest.approx(2.0)
    assert r.profile_attention_ms == pytest.approx(2.0)
    assert r.profile_final_logits_ms == pytest.approx(2.0)
    assert r.profile_layer_norm_ms == 0.0 and r.profile_tokenization_ms == 0.0
    assert r.time_to_first_token_ms == pytest.approx(10.0)
    # zero durations give zero rates, not a division error (src/main.rs:4147-4153)
    z = ex.average_row("hip", False, None, "<aggregate>", 0, 0.0, [_stats(0, 0.0, 0.0, None)], [])
    assert z.decode_tokens_per_second == 0.0 and z.total_tokens_per_second == 0.0
    assert z.time_to_first_token_ms is None


def test_csv_rows_follow_the_reference_formats():
    stats = [_stats(4, 0.010, 0.020), _stats(4, 0.030, 0.060)]
    rows = [ex.average_row("hip", True, 3, 'say "hi", twice', 4, 0.25, stats, []),
            ex.average_row("hip", False, None, "<aggregate>", 4, 0.25, [_stats(0, 0.0, 0.0, None)], [])]
    lines = ex.format_csv(rows).splitlines()
    assert lines[0] == REFERENCE_CSV_HEADER and len(lines) == 3
    assert lines[1].startswith('hip,3,"say ""hi"", twice",0,0,0,0,0,0,0,0,true,4,2,7,4.000,250.000,0.000,20.000,10.000,40.000,60.000,')
    # no prompt index and no first token: empty fields
    assert lines[2].startswith("hip,,<aggregate>,0,0,0,0,0,0,0,0,false,4,1,7,0.000,250.000,0.000,0.000,,0.000,0.000,")
    import csv
    parsed = list(csv.reader(lines))
    assert all(len(p) == len(ex.CSV_COLUMNS) for p in parsed)
    assert parsed[1][2] == 'say "hi", twice'
    table = ex.format_table(rows).splitlines()
    assert table[0].split()[:4] == ["backend", "prompt", "threads", "dense_th"]
    assert table[1].split()[:5] == ["hip", "3", "0", "0", "int8"] and table[2].split()[1] == "all"


def test_runs_must_be_positive():
    with pytest.raises(ValueError, match="runs must be > 0"):
        ex.run_experiment(None, [[1]], [1], 0)


def _c128():
    cfg = synth.Gpt2Config(vocab_size=131, n_positions=40, n_embd=128, n_layer=2, n_head=2)
    return cfg, synth.random_weights(cfg, 0x5EED0231, perturb=True)


@pytest.mark.gpu
def test_profiled_stream_matches_the_plain_stream_and_fills_the_buckets():
    cfg, w = _c128()
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w)
    ids = list(synth.token_ids(9, 0x70C00231, cfg.vocab_size))
    gen = TextGenerationConfig(max_new_tokens=12)
    plain, st = model.stream_token_ids_with_stats(ids, gen)
    got, pst, prof = model.stream_token_ids_with_stats(ids, gen, profiled=True)
    want = ref.stream_token_ids_with_stats(ids, 12, None)[0]
    assert got == plain == want
    assert pst.prompt_tokens == 9 and pst.generated_tokens == st.generated_tokens == 12
    op = [prof.qkv_projection, prof.attention, prof.attention_projection, prof.mlp_fc_projection,
          prof.mlp_projection, prof.final_logits]
    assert all(v > 0.0 for v in op)
    assert prof.layer_norm == prof.tokenization == prof.decoding == 0.0
    # the spans lie inside the run they were taken from
    assert sum(op) <= pst.prefill_time + pst.decode_time
    # sampled streams draw the same tokens either way (same logits, same generator)
    samp = TextGenerationConfig(max_new_tokens=10, temperature=0.9, top_k=20, seed=7)
    assert model.stream_token_ids_with_stats(ids, samp)[0] == \
        model.stream_token_ids_with_stats(ids, samp, profiled=True)[0]
    # the context limit and the error surface are those of the plain stream
    long = TextGenerationConfig(max_new_tokens=100)
    toks, lst, _ = model.stream_token_ids_with_stats(ids, long, profiled=True)
    assert len(toks) == cfg.n_positions and lst.generated_tokens == cfg.n_positions - 9
    from puppygrad_amd import Gpt2Error
    with pytest.raises(Gpt2Error, match="exceeds vocab_size"):
        model.stream_token_ids_with_stats([1, 999], gen, profiled=True)
    with pytest.raises(Gpt2Error, match="input_ids must not be empty"):
        model.stream_token_ids_with_stats([], gen, profiled=True)


@pytest.mark.gpu
def test_profiled_stream_of_the_persistent_path_is_taken_from_its_own_time_stamps():
    """A GPT-2 width: decode forwards run on the persistent kernel, and the profiled stream takes
    its buckets from that kernel's own time stamps (one launch per forward) and from events
    between the launches of the GEMM prefill: same tokens as the plain stream and the oracle,
    greedy and sampled, every operation bucket filled, and the spans inside the run."""
    cfg = synth.Gpt2Config(vocab_size=523, n_positions=96, n_embd=768, n_layer=3, n_head=12)
    w = synth.random_weights(cfg, 0x5EED0233, std=0.08, perturb=True)
    model, ref = Gpt2Model.new(cfg, w), oracle.Model(cfg, w, oracle.rust_config(8))
    assert "decode=persistent" in model.describe()
    ids = list(synth.token_ids(20, 0x70C00233, cfg.vocab_size))
    gen = TextGenerationConfig(max_new_tokens=16)
    plain, _ = model.stream_token_ids_with_stats(ids, gen)
    got, pst, prof = model.stream_token_ids_with_stats(ids, gen, profiled=True)
    want, _, logits, gaps = ref.stream_token_ids_with_stats(ids, 16, None, want_logits=True)
    assert got == plain
    if (gaps > 2 * (1e-4 + 1e-3 * np.abs(logits).max())).all():
        assert got == want
    op = [prof.qkv_projection, prof.attention, prof.attention_projection, prof.mlp_fc_projection,
          prof.mlp_projection, prof.final_logits]
    assert all(v > 0.0 for v in op), op
    assert prof.layer_norm >= 0.0 and prof.tokenization == prof.decoding == 0.0
    assert sum(op) + prof.layer_norm <= pst.prefill_time + pst.decode_time
    # 15 decode forwards of a few tens of microseconds each, plus the prefill's launches
    assert 15 * 10e-6 < sum(op) < 15 * 2e-3 + 5e-3, op
    samp = TextGenerationConfig(max_new_tokens=10, temperature=0.9, top_k=20, seed=7)
    assert model.stream_token_ids_with_stats(ids, samp)[0] == \
        model.stream_token_ids_with_stats(ids, samp, profiled=True)[0]
    toks, lst, _ = model.stream_token_ids_with_stats(ids, TextGenerationConfig(max_new_tokens=200), profiled=True)
    assert len(toks) == cfg.n_positions and lst.generated_tokens == cfg.n_positions - 20


@pytest.mark.gpu
def test_experiment_rows_on_the_device():
    cfg, w = _c128()
    model = Gpt2Model.new(cfg, w)
    prompts = [list(synth.token_ids(n, 0x70C00232 + n, cfg.vocab_size)) for n in (5, 20)]
    rows = ex.run_experiment(model, prompts, [4, 30], runs=3, warmup_runs=1, load_time=0.5,
                             eos_token_id=None)
    assert [(r.prompt_index, r.max_new_tokens) for r in rows] == \
        [(0, 4), (1, 4), (None, 4), (0, 30), (1, 30), (None, 30)]
    assert [r.runs for r in rows] == [3, 3, 6, 3, 3, 6]
    assert [r.prompt_tokens for r in rows[:2]] == [5, 20]
    # 30 new tokens after 20 prompt ids stop at n_positions = 40
    assert [r.generated_tokens for r in rows] == [4.0, 4.0, 4.0, 30.0, 20.0, 25.0]
    for r in rows:
        assert r.backend == "hip" and not r.quantized_weights and r.threads == 0
        assert r.decode_ms_min <= r.decode_ms_median <= r.decode_ms_p95 <= r.decode_ms_max
        assert r.decode_tokens_per_second == pytest.approx(r.generated_tokens / (r.decode_ms / 1e3))
        assert r.total_generation_ms == pytest.approx(r.prefill_ms + r.decode_ms)
        assert r.profile_qkv_projection_ms > 0 and r.profile_final_logits_ms > 0
    assert len(ex.format_csv(rows).splitlines()) == 7
    np.testing.assert_allclose(rows[2].decode_ms, (rows[0].decode_ms + rows[1].decode_ms) / 2, rtol=1e-9)
