"""GPT-2 experiment rows for the HIP backend in the reference's schema.

`puppygrad gpt2-experiment` (run_gpt2_experiment, src/main.rs:3440-3541) times repeated
generations per prompt and token budget and prints one Gpt2ExperimentRow
(src/main.rs:3356-3402) per combination, as a table, CSV or JSON; the CSV is what
benchmarks/gpt2_experiment_history.csv collects.  This module produces the same rows for
`Gpt2Model` so that GPU and CPU rows sit in one table: same columns, same order, same
averaging (average_gpt2_experiment_row, src/main.rs:3782-3897), the same distribution
summary (value_distribution / percentile, src/main.rs:4064-4111) and the same number
formats (print_gpt2_experiment_csv, src/main.rs:3933-4008).

Columns that describe the CPU thread pool (threads, dense_parallel_threshold and the
chunk sizes) have no meaning here and are 0.  The timing columns come from the normal
generation path (one persistent kernel launch per token, GEMM prefill); the nine
profile_*_ms columns come from extra passes of the same generation run as one launch per
operation and timed with HIP events, because the fused kernel has no operation
boundaries to time.

    python -m puppygrad_amd.experiment --model small --prompt-tokens 32 \
        --max-new-tokens 16,128 --runs 5 --format csv
"""
from __future__ import annotations

import argparse
import dataclasses
import json
import math
import sys
import time
from dataclasses import dataclass
from typing import Iterable, List, Optional, Sequence

from . import _lib, synth
from .gpt2 import (GPT2_EOS_TOKEN_ID, GenerationStats, Gpt2Config, Gpt2HipConfig, Gpt2Model,
                   Gpt2OperationProfile, TextGenerationConfig)
from .runtime import Gpt2Runtime


@dataclass
class Gpt2ExperimentRow:
    """Gpt2ExperimentRow (src/main.rs:3356-3402): field order is the CSV column order."""
    backend: str
    prompt_index: Optional[int]
    prompt: str
    threads: int
    dense_parallel_threshold: int
    qkv_chunk_size: int
    attention_projection_chunk_size: int
    mlp_fc_chunk_size: int
    mlp_projection_chunk_size: int
    logits_chunk_size: int
    attention_head_parallel_threshold: int
    quantized_weights: bool
    max_new_tokens: int
    runs: int
    prompt_tokens: int
    generated_tokens: float
    load_ms: float
    tokenize_ms: float
    prefill_ms: float
    time_to_first_token_ms: Optional[float]
    decode_ms: float
    total_generation_ms: float
    decode_ms_min: float
    decode_ms_median: float
    decode_ms_p95: float
    decode_ms_max: float
    decode_ms_stddev: float
    total_generation_ms_min: float
    total_generation_ms_median: float
    total_generation_ms_p95: float
    total_generation_ms_max: float
    total_generation_ms_stddev: float
    prefill_tokens_per_second: float
    decode_tokens_per_second: float
    total_tokens_per_second: float
    profile_tokenization_ms: float
    profile_layer_norm_ms: float
    profile_qkv_projection_ms: float
    profile_attention_ms: float
    profile_attention_projection_ms: float
    profile_mlp_fc_projection_ms: float
    profile_mlp_projection_ms: float
    profile_final_logits_ms: float
    profile_decoding_ms: float


CSV_COLUMNS = [f.name for f in dataclasses.fields(Gpt2ExperimentRow)]


@dataclass
class DistributionSummary:
    min: float = 0.0
    p25: float = 0.0
    median: float = 0.0
    p95: float = 0.0
    max: float = 0.0
    stddev: float = 0.0


def percentile(sorted_values: Sequence[float], p: float) -> float:
    """Linear interpolation between the two nearest ranks (src/main.rs:4099-4111)."""
    if not sorted_values:
        return 0.0
    rank = min(max(p, 0.0), 1.0) * (len(sorted_values) - 1)
    lower, upper = math.floor(rank), math.ceil(rank)
    if lower == upper:
        return sorted_values[lower]
    weight = rank - lower
    return sorted_values[lower] * (1.0 - weight) + sorted_values[upper] * weight


def value_distribution(values: Iterable[float]) -> DistributionSummary:
    """min / quartile / median / p95 / max and the population standard deviation
    (src/main.rs:4064-4097)."""
    v = sorted(values)
    if not v:
        return DistributionSummary()
    mean = sum(v) / len(v)
    variance = sum((x - mean) ** 2 for x in v) / len(v)
    return DistributionSummary(v[0], percentile(v, 0.25), percentile(v, 0.5), percentile(v, 0.95),
                               v[-1], math.sqrt(variance))


def _mean(values: Sequence[float]) -> float:
    return sum(values) / len(values) if values else 0.0


def _rate(tokens: float, seconds: float) -> float:
    return 0.0 if seconds == 0.0 else tokens / seconds


def average_row(backend: str, quantized_weights: bool, prompt_index: Optional[int], prompt: str,
                max_new_tokens: int, load_time: float, stats: Sequence[GenerationStats],
                profiles: Sequence[Gpt2OperationProfile]) -> Gpt2ExperimentRow:
    """average_gpt2_experiment_row (src/main.rs:3782-3897): means over the runs, rates from
    the mean times.  Times are seconds on the way in, milliseconds in the row."""
    runs = len(stats)
    generated = _mean([float(s.generated_tokens) for s in stats])
    prefill = _mean([s.prefill_time for s in stats])
    decode = _mean([s.decode_time for s in stats])
    total = _mean([s.total_generation_time for s in stats])
    first = [s.first_token_time for s in stats if s.first_token_time is not None]
    dsum = value_distribution(s.decode_time * 1e3 for s in stats)
    tsum = value_distribution(s.total_generation_time * 1e3 for s in stats)
    prompt_tokens = stats[0].prompt_tokens if stats else 0
    bucket = lambda name: _mean([getattr(p, name) for p in profiles]) * 1e3
    return Gpt2ExperimentRow(
        backend=backend, prompt_index=prompt_index, prompt=prompt, threads=0,
        dense_parallel_threshold=0, qkv_chunk_size=0, attention_projection_chunk_size=0,
        mlp_fc_chunk_size=0, mlp_projection_chunk_size=0, logits_chunk_size=0,
        attention_head_parallel_threshold=0, quantized_weights=quantized_weights,
        max_new_tokens=max_new_tokens, runs=runs, prompt_tokens=prompt_tokens,
        generated_tokens=generated, load_ms=load_time * 1e3, tokenize_ms=_mean([getattr(s, "tokenize_time", 0.0) for s in stats]) * 1e3,
        prefill_ms=prefill * 1e3, time_to_first_token_ms=_mean(first) * 1e3 if first else None,
        decode_ms=decode * 1e3, total_generation_ms=total * 1e3,
        decode_ms_min=dsum.min, decode_ms_median=dsum.median, decode_ms_p95=dsum.p95,
        decode_ms_max=dsum.max, decode_ms_stddev=dsum.stddev,
        total_generation_ms_min=tsum.min, total_generation_ms_median=tsum.median,
        total_generation_ms_p95=tsum.p95, total_generation_ms_max=tsum.max,
        total_generation_ms_stddev=tsum.stddev,
        prefill_tokens_per_second=_rate(float(prompt_tokens), prefill),
        decode_tokens_per_second=_rate(generated, decode),
        total_tokens_per_second=_rate(prompt_tokens + generated, total),
        profile_tokenization_ms=bucket("tokenization"), profile_layer_norm_ms=bucket("layer_norm"),
        profile_qkv_projection_ms=bucket("qkv_projection"), profile_attention_ms=bucket("attention"),
        profile_attention_projection_ms=bucket("attention_projection"),
        profile_mlp_fc_projection_ms=bucket("mlp_fc_projection"),
        profile_mlp_projection_ms=bucket("mlp_projection"),
        profile_final_logits_ms=bucket("final_logits"), profile_decoding_ms=bucket("decoding"))


def load_experiment_prompts(prompt: Optional[str], prompt_file: Optional[str]) -> List[str]:
    """load_experiment_prompts (src/main.rs:4009-4030): the non-empty trimmed lines of the
    file, or the one prompt."""
    if prompt_file is not None:
        try:
            with open(prompt_file, encoding="utf-8") as f:
                text = f.read()
        except OSError as e:
            raise ValueError(f"failed to read --prompt-file {prompt_file}: {e}")
        prompts = [line.strip() for line in text.splitlines() if line.strip()]
        if not prompts:
            raise ValueError(f"--prompt-file {prompt_file} contains no prompts")
        return prompts
    if prompt is None:
        raise ValueError("experiment gpt2 requires --prompt or --prompt-file")
    return [prompt]


def run_experiment(model, prompts: Sequence, token_counts: Sequence[int], runs: int,
                   warmup_runs: int = 0, load_time: float = 0.0, profile_runs: int = 1,
                   quantized_weights: bool = False,
                   prompt_labels: Optional[Sequence[str]] = None,
                   eos_token_id: Optional[int] = GPT2_EOS_TOKEN_ID) -> List[Gpt2ExperimentRow]:
    """The loops of run_gpt2_experiment (src/main.rs:3478-3527): per token budget and prompt,
    `warmup_runs` untimed generations, `runs` timed ones and `profile_runs` profiled ones; one
    row per prompt, plus an "<aggregate>" row over all of them when there are several prompts.
    `model` is a Gpt2Model with prompts given as token ids, or a Gpt2Runtime with prompts given
    as text (then the tokenizer's and the text streamer's host time are in the rows, as in the
    reference, which runs stream_greedy_text_with_stats).  Generation is greedy with GPT-2's EOS
    id (Gpt2GenerationConfig::new, src/models/gpt2/options.rs:156-162) unless another, or None,
    is given."""
    if runs == 0:
        raise ValueError("experiment --runs must be > 0")
    text = hasattr(model, "tokenizer")
    if text:
        runtime = model

        class _Text:  # the id-prompt interface over the runtime's text entry point
            @staticmethod
            def stream_token_ids_with_stats(prompt, generation, profiled=False):
                out = runtime.stream_text_with_stats(prompt, generation, lambda _t: None, profiled)
                return out if profiled else out[:2]
        model = _Text
    labels = list(prompt_labels) if prompt_labels is not None else [
        p if text else f"<{len(p)} token ids>" for p in prompts]
    rows = []
    for max_new in token_counts:
        generation = TextGenerationConfig(max_new, eos_token_id=eos_token_id)
        generation.validate()
        all_stats, all_profiles = [], []
        for index, prompt in enumerate(prompts):
            for _ in range(warmup_runs):
                model.stream_token_ids_with_stats(prompt, generation)
            stats = [model.stream_token_ids_with_stats(prompt, generation)[1] for _ in range(runs)]
            profiles = [model.stream_token_ids_with_stats(prompt, generation, profiled=True)[2]
                        for _ in range(profile_runs)]
            all_stats += stats
            all_profiles += profiles
            rows.append(average_row("hip", quantized_weights, index, labels[index], max_new,
                                    load_time, stats, profiles))
        if len(prompts) > 1:
            rows.append(average_row("hip", quantized_weights, None, "<aggregate>", max_new,
                                    load_time, all_stats, all_profiles))
    return rows


def csv_escape(value: str) -> str:
    """src/main.rs:4032-4038."""
    if "," in value or '"' in value or "\n" in value:
        return '"' + value.replace('"', '""') + '"'
    return value


def format_csv(rows: Sequence[Gpt2ExperimentRow]) -> str:
    """print_gpt2_experiment_csv (src/main.rs:3933-4008): header, then per row the
    configuration columns as they are and every measured column with three decimals; an
    absent prompt index or first-token time is an empty field."""
    lines = [",".join(CSV_COLUMNS)]
    for row in rows:
        out = []
        for name in CSV_COLUMNS:
            v = getattr(row, name)
            if v is None:
                out.append("")
            elif isinstance(v, bool):
                out.append("true" if v else "false")
            elif isinstance(v, float):
                out.append(f"{v:.3f}")
            elif isinstance(v, str):
                out.append(csv_escape(v))
            else:
                out.append(str(v))
        lines.append(",".join(out))
    return "\n".join(lines) + "\n"


def format_table(rows: Sequence[Gpt2ExperimentRow]) -> str:
    """print_gpt2_experiment_table (src/main.rs:3899-3931)."""
    head = ("backend", "prompt", "threads", "dense_th", "weights", "new_tok", "runs", "prompt", "gen",
            "load_ms", "prefill", "dec_avg", "dec_p95", "dec_sd", "tok/s", "total/s")
    fmt_h = "{:<7} {:>6} {:>7} {:>9} {:>7} {:>8} {:>5} {:>7} {:>7} {:>8} {:>8} {:>8} {:>8} {:>8} {:>10} {:>10}"
    fmt_r = ("{:<7} {:>6} {:>7} {:>9} {:>7} {:>8} {:>5} {:>7} {:>7.1f} {:>8.1f} {:>8.1f} {:>8.1f} "
             "{:>8.1f} {:>8.1f} {:>10.2f} {:>10.2f}")
    lines = [fmt_h.format(*head)]
    for r in rows:
        lines.append(fmt_r.format(
            r.backend, "all" if r.prompt_index is None else str(r.prompt_index), r.threads,
            r.dense_parallel_threshold, "int8" if r.quantized_weights else "f32", r.max_new_tokens,
            r.runs, r.prompt_tokens, r.generated_tokens, r.load_ms, r.prefill_ms, r.decode_ms,
            r.decode_ms_p95, r.decode_ms_stddev, r.decode_tokens_per_second,
            r.total_tokens_per_second))
    return "\n".join(lines) + "\n"


def format_json(rows: Sequence[Gpt2ExperimentRow]) -> str:
    return json.dumps([dataclasses.asdict(r) for r in rows], indent=2) + "\n"


def _usize_list(name: str, text: str) -> List[int]:
    """parse_usize_list (src/main.rs:4040-4056)."""
    try:
        out = [int(v) for v in (t.strip() for t in text.split(",")) if v]
    except ValueError as e:
        raise SystemExit(f"invalid --{name} value: {e}")
    if not out or any(v < 0 for v in out):
        raise SystemExit(f"--{name} must contain at least one value")
    return out


def main(argv: Optional[Sequence[str]] = None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", choices=["small", "medium", "large", "xl"], default="small",
                    help="architecture for seeded random weights (ignored with --model-dir)")
    ap.add_argument("--model-dir", help="directory with config.json and model.safetensors")
    ap.add_argument("--prompt-tokens", default="32",
                    help="comma-separated prompt lengths; ids are seeded uniform draws")
    ap.add_argument("--prompt", help="text prompt (needs --model-dir with a tokenizer.json)")
    ap.add_argument("--prompt-file", help="one text prompt per line (needs --model-dir)")
    ap.add_argument("--max-new-tokens", default="16")
    ap.add_argument("--runs", type=int, default=3)
    ap.add_argument("--warmup-runs", type=int, default=1)
    ap.add_argument("--profile-runs", type=int, default=1)
    ap.add_argument("--quantized-weights", action="store_true", help="int8 rows (QuantizedRows)")
    ap.add_argument("--format", choices=["table", "csv", "json"], default="table")
    args = ap.parse_args(argv)
    if args.runs == 0:
        raise SystemExit("experiment --runs must be > 0")
    hip = Gpt2HipConfig(weight_storage=_lib.PG_STORE_INT8 if args.quantized_weights
                        else _lib.PG_STORE_F32)
    text_prompts = None
    if args.prompt is not None or args.prompt_file is not None:
        if not args.model_dir:
            raise SystemExit("--prompt / --prompt-file need --model-dir (tokenizer.json)")
        try:
            text_prompts = load_experiment_prompts(args.prompt, args.prompt_file)
        except ValueError as e:
            raise SystemExit(str(e))
    t0 = time.perf_counter()
    if text_prompts is not None:
        model = Gpt2Runtime.from_dir(args.model_dir, hip)
    elif args.model_dir:
        model = Gpt2Model.from_dir(args.model_dir, hip)
    else:
        kw = {"small": synth.GPT2_SMALL, "medium": synth.GPT2_MEDIUM, "large": synth.GPT2_LARGE,
              "xl": synth.GPT2_XL}[args.model]
        cfg = Gpt2Config(**kw)
        model = Gpt2Model.new(cfg, synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 1), hip)
    load_time = time.perf_counter() - t0
    core = model.model if text_prompts is not None else model
    print(f"loaded GPT-2 with {core.describe()}", file=sys.stderr)
    vocab = core.config.vocab_size
    prompts = text_prompts if text_prompts is not None else [
        list(synth.token_ids(n, synth.TOKEN_SEED_BASE + 1, vocab))
        for n in _usize_list("prompt-tokens", args.prompt_tokens)]
    rows = run_experiment(model, prompts, _usize_list("max-new-tokens", args.max_new_tokens),
                          args.runs, args.warmup_runs, load_time, args.profile_runs,
                          args.quantized_weights)
    sys.stdout.write({"table": format_table, "csv": format_csv, "json": format_json}[args.format](rows))
    return 0


if __name__ == "__main__":
    sys.exit(main())
