"""Autotune of the HIP backend's tunables in the reference's shape.

`puppygrad autotune gpt2` (src/models/autotune.rs:1-85, run_gpt2_autotune in
src/main.rs:2732-2807) builds the model once per candidate configuration, streams greedy
generations for every prompt, scores a candidate by its median decode tokens per second,
validates the best one with more runs and saves it to `{model_dir}/puppygrad-tune.json`
(SavedGpt2Tuning, src/main.rs:2611-2623), which later runs load (load_gpt2_tuning,
src/main.rs:2564-2586).  This module does the same over the tunables of `Gpt2HipConfig`
(the counterpart of the thresholds and chunk sizes of `Gpt2RustConfig`): keys per attention
item of the fused decode kernel, attention blocks per CU of the per-operation / batched
decode attention, and three knobs of the GEMM prefill's planner: work items per CU of the
split-K tile GEMM, the row count from which f32 products move to the bf16 matrix cores, and the
prompt length from which the GEMM prefill is used at all.  The decode knobs move the reference's
score (median decode tokens per second); the planner's knobs only move the prompt's share of a
generation, so `--score total` (median of prompt + generated tokens over the whole generation
time, a figure the reference's measurement already holds) or `--score prefill` ranks by that
instead.  The saved file has the reference's fields with a `hip` object in the place of `rust`;
`Gpt2Model.from_dir` (pg_gpt2_create_from_dir) reads it.

    python -m puppygrad_amd.autotune --model medium --prompt-tokens 128 --max-new-tokens 64 \
        --save-tuning puppygrad-tune.json
"""
from __future__ import annotations

import argparse
import dataclasses
import itertools
import json
import sys
import time
from dataclasses import dataclass, field
from pathlib import Path
from typing import Callable, Generic, List, Optional, Protocol, Sequence, TypeVar

from . import _lib, synth
from .experiment import _rate, _usize_list, value_distribution
from .gpt2 import (GPT2_EOS_TOKEN_ID, GenerationStats, Gpt2Config, Gpt2HipConfig, Gpt2Model,
                   TextGenerationConfig)

C = TypeVar("C")
M = TypeVar("M")


@dataclass
class AutoTuneOptions:
    """AutoTuneOptions (src/models/autotune.rs:1-17)."""
    warmup_runs: int = 1
    measured_runs: int = 3
    max_trials: Optional[int] = None


@dataclass
class AutoTuneTrial(Generic[C, M]):
    """AutoTuneTrial (autotune.rs:19-24)."""
    config: C
    measurement: M
    score: float


@dataclass
class AutoTuneResult(Generic[C, M]):
    """AutoTuneResult (autotune.rs:26-31)."""
    best_config: C
    best_score: float
    trials: List[AutoTuneTrial]


class AutoTuneTarget(Protocol):
    """AutoTuneTarget (autotune.rs:33-48)."""

    def candidate_configs(self) -> list: ...

    def evaluate_config(self, config, options: AutoTuneOptions): ...

    def score(self, measurement) -> float: ...


def autotune(target: AutoTuneTarget, options: AutoTuneOptions) -> AutoTuneResult:
    """autotune (autotune.rs:50-85): every candidate (the first max_trials of them) is
    evaluated once; the first one with the strictly greatest score wins."""
    candidates = list(target.candidate_configs())
    if options.max_trials is not None:
        candidates = candidates[:options.max_trials]
    trials: List[AutoTuneTrial] = []
    best_index, best_score = None, float("-inf")
    for config in candidates:
        measurement = target.evaluate_config(config, options)
        score = target.score(measurement)
        if score > best_score:
            best_score, best_index = score, len(trials)
        trials.append(AutoTuneTrial(config, measurement, score))
    if best_index is None:
        raise ValueError("autotune requires at least one candidate")
    return AutoTuneResult(trials[best_index].config, best_score, trials)


@dataclass
class Gpt2AutoTuneMeasurement:
    """Gpt2AutoTuneMeasurement (src/main.rs:2593-2609)."""
    load_ms: float = 0.0
    prompt_count: int = 0
    runs_per_prompt: int = 0
    generated_tokens: int = 0
    decode_tokens_per_second: float = 0.0
    decode_tokens_per_second_p25: float = 0.0
    decode_tokens_per_second_median: float = 0.0
    decode_tokens_per_second_p95: float = 0.0
    decode_tokens_per_second_stddev: float = 0.0
    total_tokens_per_second: float = 0.0
    total_tokens_per_second_median: float = 0.0
    prefill_tokens_per_second_median: float = 0.0  # (not in the reference's struct: for --score prefill)
    prefill_ms: float = 0.0
    decode_ms: float = 0.0
    total_generation_ms: float = 0.0


def summarize_runs(load_time: float, prompt_count: int, runs_per_prompt: int,
                   stats: Sequence[GenerationStats]) -> Gpt2AutoTuneMeasurement:
    """The arithmetic of evaluate_config (src/main.rs:2685-2724) on the collected stats."""
    generated = sum(s.generated_tokens for s in stats)
    prompt_tokens = sum(s.prompt_tokens for s in stats)
    prefill = sum(s.prefill_time for s in stats)
    decode = sum(s.decode_time for s in stats)
    total = sum(s.total_generation_time for s in stats)
    decode_tps = value_distribution(_rate(float(s.generated_tokens), s.decode_time) for s in stats)
    total_tps = value_distribution(
        _rate(float(s.prompt_tokens + s.generated_tokens), s.total_generation_time) for s in stats)
    prefill_tps = value_distribution(_rate(float(s.prompt_tokens), s.prefill_time) for s in stats)
    n = max(len(stats), 1)
    return Gpt2AutoTuneMeasurement(
        load_ms=load_time * 1e3, prompt_count=prompt_count, runs_per_prompt=runs_per_prompt,
        generated_tokens=generated, decode_tokens_per_second=_rate(float(generated), decode),
        decode_tokens_per_second_p25=decode_tps.p25, decode_tokens_per_second_median=decode_tps.median,
        decode_tokens_per_second_p95=decode_tps.p95, decode_tokens_per_second_stddev=decode_tps.stddev,
        total_tokens_per_second=_rate(float(prompt_tokens + generated), total),
        total_tokens_per_second_median=total_tps.median,
        prefill_tokens_per_second_median=prefill_tps.median, prefill_ms=prefill * 1e3 / n,
        decode_ms=decode * 1e3 / n, total_generation_ms=total * 1e3 / n)


TUNABLES = ("attn_item_keys", "attn_blocks_per_cu", "gemm_split_items_per_cu", "gemm_b9_min_rows",
            "seq_gemm_min_tokens")
SCORES = {"decode": ("median_decode_tokens_per_second", "decode_tokens_per_second_median"),
          "total": ("median_total_tokens_per_second", "total_tokens_per_second_median"),
          "prefill": ("median_prefill_tokens_per_second", "prefill_tokens_per_second_median")}


def candidate_grid(base: Gpt2HipConfig, attn_item_keys: Sequence[int], attn_blocks_per_cu: Sequence[int],
                   gemm_split_items_per_cu: Sequence[int], gemm_b9_min_rows: Sequence[int] = (0,),
                   seq_gemm_min_tokens: Sequence[int] = (0,)) -> List[Gpt2HipConfig]:
    """gpt2_autotune_candidates (src/main.rs:2809-2873): the cross product of the value
    lists, the first list varying slowest."""
    out = []
    for keys, blocks, items, b9, seq in itertools.product(attn_item_keys, attn_blocks_per_cu,
                                                          gemm_split_items_per_cu, gemm_b9_min_rows,
                                                          seq_gemm_min_tokens):
        out.append(dataclasses.replace(base, attn_item_keys=keys, attn_blocks_per_cu=blocks,
                                       gemm_split_items_per_cu=items, gemm_b9_min_rows=b9,
                                       seq_gemm_min_tokens=seq))
    if not out:
        raise ValueError("autotune gpt2 generated no candidates")
    return out


@dataclass
class Gpt2AutoTuneTarget:
    """Gpt2AutoTuneTarget (src/main.rs:2625-2730).  `make_model(hip_config)` stands where
    Gpt2Runtime::from_dir_with_backend does; prompts are token-id lists."""
    make_model: Callable[[Gpt2HipConfig], Gpt2Model]
    prompts: Sequence[Sequence[int]]
    max_new_tokens: int
    candidates: List[Gpt2HipConfig]
    log: Callable[[str], None] = lambda line: print(line, file=sys.stderr)
    eos_token_id: Optional[int] = GPT2_EOS_TOKEN_ID  # Gpt2GenerationConfig::new; None for small vocabularies
    score_by: str = "decode"  # key of SCORES; the reference scores by decode

    def candidate_configs(self) -> List[Gpt2HipConfig]:
        return list(self.candidates)

    def evaluate_config(self, config: Gpt2HipConfig, options: AutoTuneOptions) -> Gpt2AutoTuneMeasurement:
        self.log("autotune trial: " + " ".join(f"{k}={getattr(config, k)}" for k in TUNABLES))
        t0 = time.perf_counter()
        model = self.make_model(config)
        load_time = time.perf_counter() - t0
        generation = TextGenerationConfig(self.max_new_tokens, eos_token_id=self.eos_token_id)
        generation.validate()
        stats: List[GenerationStats] = []
        for prompt in self.prompts:
            for _ in range(options.warmup_runs):
                model.stream_token_ids_with_stats(prompt, generation)
            for _ in range(options.measured_runs):
                stats.append(model.stream_token_ids_with_stats(prompt, generation)[1])
        return summarize_runs(load_time, len(self.prompts), options.measured_runs, stats)

    def score(self, measurement: Gpt2AutoTuneMeasurement) -> float:
        return getattr(measurement, SCORES[self.score_by][1])


def save_gpt2_tuning(path, best_config: Gpt2HipConfig, search_score: float, validation_score: float,
                     validation_measurement: Gpt2AutoTuneMeasurement, max_new_tokens: int,
                     options: AutoTuneOptions, model: str = "gpt2", score_by: str = "decode") -> None:
    """save_gpt2_tuning (src/main.rs:2927-2958): SavedGpt2Tuning as pretty JSON."""
    saved = {
        "model": model, "backend": "hip", "score_name": SCORES[score_by][0],
        "score": validation_score, "search_score": search_score, "max_new_tokens": max_new_tokens,
        "warmup_runs": options.warmup_runs, "measured_runs": options.measured_runs,
        "prompt_count": validation_measurement.prompt_count,
        "hip": {k: int(getattr(best_config, k)) for k in TUNABLES},
        "measurement": dataclasses.asdict(validation_measurement),
    }
    path = Path(path)
    path.parent.mkdir(parents=True, exist_ok=True)
    path.write_text(json.dumps(saved, indent=2) + "\n")


def load_gpt2_tuning(tuning_file, model_dir=None, base: Optional[Gpt2HipConfig] = None) -> Optional[Gpt2HipConfig]:
    """load_gpt2_tuning (src/main.rs:2564-2586): the named file, or
    {model_dir}/puppygrad-tune.json when it exists; None when there is no default file.
    Tunables `base` sets explicitly (non-zero) are kept."""
    import ctypes
    explicit = tuning_file is not None
    path = Path(tuning_file) if explicit else Path(model_dir) / "puppygrad-tune.json"
    if not path.exists():
        if explicit:
            raise FileNotFoundError(f"tuning file {path} does not exist")
        return None
    cfg = base or Gpt2HipConfig()
    opts = cfg.to_c()
    found = ctypes.c_int32(0)
    from .gpt2 import _check
    _check(_lib.load().pg_hip_load_tuning(str(path).encode(), ctypes.byref(opts), ctypes.byref(found)))
    return dataclasses.replace(cfg, **{k: int(getattr(opts, k)) for k in TUNABLES})


def run_gpt2_autotune(make_model, prompts, max_new_tokens: int, candidates: List[Gpt2HipConfig],
                      options: AutoTuneOptions, validation_runs: int, save_path=None, model_name="gpt2",
                      log=lambda line: print(line, file=sys.stderr), eos_token_id=GPT2_EOS_TOKEN_ID,
                      score_by: str = "decode"):
    """run_gpt2_autotune (src/main.rs:2732-2807): scan, validate the winner, save it."""
    if options.measured_runs == 0:
        raise ValueError("autotune gpt2 --runs must be > 0")
    if options.max_trials is not None and options.max_trials == 0:
        raise ValueError("autotune gpt2 --max-trials must be > 0")
    log(f"autotune: {len(candidates)} candidates, evaluating up to "
        f"{options.max_trials if options.max_trials is not None else len(candidates)}")
    if score_by not in SCORES:
        raise ValueError(f"autotune gpt2 --score must be one of {', '.join(SCORES)}")
    target = Gpt2AutoTuneTarget(make_model, prompts, max_new_tokens, candidates, log, eos_token_id, score_by)
    result = autotune(target, options)
    validation_options = AutoTuneOptions(options.warmup_runs, validation_runs, None)
    log(f"validating best config with {validation_runs} measured runs")
    validation = target.evaluate_config(result.best_config, validation_options)
    validation_score = target.score(validation)
    if save_path is not None:
        save_gpt2_tuning(save_path, result.best_config, result.best_score, validation_score, validation,
                         max_new_tokens, validation_options, model_name, score_by)
        log(f"saved tuning config to {save_path}")
    return result, validation, validation_score


def main(argv: Optional[Sequence[str]] = None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", choices=["small", "medium", "large", "xl"], default="small",
                    help="architecture for seeded random weights (ignored with --model-dir)")
    ap.add_argument("--model-dir", help="directory with config.json and model.safetensors")
    ap.add_argument("--prompt-tokens", default="32", help="comma-separated prompt lengths (seeded ids)")
    ap.add_argument("--max-new-tokens", type=int, default=64)
    ap.add_argument("--runs", type=int, default=3)
    ap.add_argument("--warmup-runs", type=int, default=1)
    ap.add_argument("--validation-runs", type=int, default=5)
    ap.add_argument("--max-trials", type=int, default=64)
    ap.add_argument("--attn-item-keys", default="128,256")
    ap.add_argument("--attn-blocks-per-cu", default="4")
    ap.add_argument("--gemm-split-items-per-cu", default="3")
    ap.add_argument("--gemm-b9-min-rows", default="0", help="0: the built-in 1024")
    ap.add_argument("--seq-gemm-min-tokens", default="0", help="0: the built-in 4")
    ap.add_argument("--score", choices=sorted(SCORES), default="decode",
                    help="what ranks the candidates (the reference: decode)")
    ap.add_argument("--quantized-weights", action="store_true")
    ap.add_argument("--save-tuning", help="default: {model-dir}/puppygrad-tune.json, or none without --model-dir")
    args = ap.parse_args(argv)
    base = Gpt2HipConfig(weight_storage=_lib.PG_STORE_INT8 if args.quantized_weights else _lib.PG_STORE_F32)
    if args.model_dir:
        make_model = lambda hip: Gpt2Model.from_dir(args.model_dir, hip)
        vocab = Gpt2Config.from_json_file(Path(args.model_dir) / "config.json").vocab_size
        save_path = args.save_tuning or Path(args.model_dir) / "puppygrad-tune.json"
    else:
        kw = {"small": synth.GPT2_SMALL, "medium": synth.GPT2_MEDIUM, "large": synth.GPT2_LARGE,
              "xl": synth.GPT2_XL}[args.model]
        cfg = Gpt2Config(**kw)
        weights = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 1)
        make_model = lambda hip: Gpt2Model.new(cfg, weights, hip)
        vocab = cfg.vocab_size
        save_path = args.save_tuning
    prompts = [list(synth.token_ids(n, synth.TOKEN_SEED_BASE + 1, vocab))
               for n in _usize_list("prompt-tokens", args.prompt_tokens)]
    candidates = candidate_grid(base, _usize_list("attn-item-keys", args.attn_item_keys),
                                _usize_list("attn-blocks-per-cu", args.attn_blocks_per_cu),
                                _usize_list("gemm-split-items-per-cu", args.gemm_split_items_per_cu),
                                _usize_list("gemm-b9-min-rows", args.gemm_b9_min_rows),
                                _usize_list("seq-gemm-min-tokens", args.seq_gemm_min_tokens))
    options = AutoTuneOptions(args.warmup_runs, args.runs, args.max_trials)
    result, validation, score = run_gpt2_autotune(make_model, prompts, args.max_new_tokens, candidates,
                                                  options, args.validation_runs, save_path,
                                                  args.model if not args.model_dir else "gpt2",
                                                  score_by=args.score)
    print("best config:")
    for k in TUNABLES:
        print(f"  --{k.replace('_', '-')} {getattr(result.best_config, k)}")
    print(f"search score ({SCORES[args.score][0]}): {result.best_score:.2f} tok/s median")
    for trial in result.trials:
        print("  trial " + " ".join(f"{k}={getattr(trial.config, k)}" for k in TUNABLES)
              + f": {trial.score:.2f} tok/s median")
    print(f"\nvalidated best: {score:.2f} tok/s median ({validation.decode_tokens_per_second:.2f} tok/s mean)")
    return 0


if __name__ == "__main__":
    sys.exit(main())
