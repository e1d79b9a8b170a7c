#!/usr/bin/env python3
"""Headline benchmark: GPT-2 XL 1.5B fp32, batch-1 greedy decode with a KV cache
prefilled to 896 tokens (the configuration the headline metric is quoted on), on one MI355X.

A step is one cached decoder forward (one token).  The timed region holds
weights, KV cache and the first logits resident in HBM; token selection
(argmax) runs on the device and only the ids return to the host afterwards.
The same invocation then measures the other configurations the metric names (124M batch-1
decode, 124M full-context prefill, 355M batch-16 and XL bf16 batch-32 decode steps) and reports
them under "secondary", each with the roofline of its own bound.
Prints ONE JSON line.  `--gpus N` with N > 1 is refused: this path runs on one GPU.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def weight_bytes(cfg, int8: bool = False, bf16: bool = False) -> int:
    """Bytes of parameters one decode step reads: every block tensor, ln_f, wte
    (as lm_head) and the two embedding rows.  With int8 storage the four block matrices
    and the lm_head are one byte per element plus one f32 scale per row; with bf16 storage
    they (and the wte embedding row) are two bytes per element."""
    C_, I, L, V = cfg.n_embd, cfg.n_inner, cfg.n_layer, cfg.vocab_size
    if int8 or bf16:
        eb = 1 if int8 else 2
        mats = eb * (3 * C_ * C_ + C_ * C_ + 2 * C_ * I)       # bytes
        scales = (3 * C_ + C_ + I + C_) if int8 else 0         # f32 each
        small = 3 * C_ + C_ + I + C_ + 4 * C_                  # biases and LayerNorm, f32
        embed = 4 * C_ + (4 if int8 else 2) * C_               # wpe row + wte row
        return L * (mats + 4 * (scales + small)) + eb * V * C_ + (4 * V if int8 else 0) + 4 * 2 * C_ + embed
    per_layer = 3 * C_ * C_ + 3 * C_ + C_ * C_ + C_ + 2 * C_ * I + I + C_ + 4 * C_
    return 4 * (L * per_layer + 2 * C_ + V * C_ + 2 * C_)


def kv_bytes(cfg, pos: int) -> int:
    """K and V rows of positions [0, pos] over all layers."""
    return 4 * 2 * cfg.n_layer * cfg.n_embd * (pos + 1)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=127)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--model", default="xl", choices=["xl", "large", "medium", "small"])
    ap.add_argument("--prefill", type=int, default=None, help="tokens in the cache before decode")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the other configurations (they run only beside the default workload)")
    ap.add_argument("--decode-path", default="auto", choices=["auto", "kernels", "persistent"])
    ap.add_argument("--workload", default="decode",
                    choices=["decode", "prefill", "batch-decode", "sampled-stream"],
                    help="prefill: a step is one prefill of --prefill tokens (GEMM path, MFMA-bound); "
                         "batch-decode: a step is one greedy step of --batch sequences; "
                         "sampled-stream: streamed generations of --steps tokens with sampled selection")
    ap.add_argument("--batch", type=int, default=None,
                    help="sequences of a batched step (batch-decode: 16 by default; prefill: 1)")
    ap.add_argument("--bf16", action="store_true", help="store the weights as bf16 (fp32 arithmetic)")
    ap.add_argument("--int8", action="store_true",
                    help="store the weights as int8 rows with f32 scales (the reference's "
                         "quantized_weights; fp32 arithmetic); --workload decode")
    args = ap.parse_args()
    args.batch_given = args.batch is not None
    if args.batch is None:
        args.batch = 16
    if args.gpus != 1:
        log("bench.py: this path runs on ONE GPU (a batch-1 decode step has one all-reduce of "
            "n_embd floats after every projection pair to offer to a second GPU: latency-bound); "
            "--gpus must be 1")
        return 2

    from puppygrad_amd import Gpt2Config, Gpt2HipConfig, Gpt2Model, _lib, synth

    model_kw = {"xl": synth.GPT2_XL, "large": synth.GPT2_LARGE, "medium": synth.GPT2_MEDIUM,
                "small": synth.GPT2_SMALL}[args.model]
    cfg_no = {"xl": 4, "large": 6, "medium": 3, "small": 1}[args.model]
    cfg = Gpt2Config(**model_kw)
    n_prefill = args.prefill if args.prefill is not None else {"xl": 896, "large": 512, "medium": 128, "small": 32}[args.model]
    room = cfg.n_positions - n_prefill  # tokens one pass can generate

    t0 = time.time()
    weights = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + cfg_no)
    ids = synth.token_ids(n_prefill, synth.TOKEN_SEED_BASE + cfg_no, cfg.vocab_size)
    log(f"[bench] synthetic weights: {time.time() - t0:.1f}s")
    t0 = time.time()
    path = {"auto": _lib.PG_DECODE_AUTO, "kernels": _lib.PG_DECODE_KERNELS,
            "persistent": _lib.PG_DECODE_PERSISTENT}[args.decode_path]
    storage = _lib.PG_STORE_BF16 if args.bf16 else _lib.PG_STORE_INT8 if args.int8 else _lib.PG_STORE_F32
    if args.int8 and (args.workload != "decode" or args.bf16):
        log("bench.py: --int8 is for --workload decode, without --bf16")
        return 2
    model = Gpt2Model.new(cfg, weights, Gpt2HipConfig(device=0, weight_storage=storage, decode_path=path))
    log(f"[bench] upload: {time.time() - t0:.1f}s; backend: {model.describe()}")

    if args.workload == "prefill":
        return bench_prefill(args, cfg, model, ids, n_prefill)
    if args.workload == "batch-decode":
        return bench_batch_decode(args, cfg, model, n_prefill)
    if args.workload == "sampled-stream":
        r = measure_sampled_stream(model, ids, min(args.steps + 1, room), name=f"GPT-2 {args.model}")
        r.update({"metric": f"streamed generation tokens/sec with sampled selection, GPT-2 {args.model} fp32 bs=1",
                  "n_gpus": 1, "higher_is_better": True, "data": "synthetic", "dtype": "f32"})
        print(json.dumps(r), flush=True)
        return 0

    d = measure_decode(model, cfg, ids, n_prefill, args.steps, args.warmup, args.int8, args.bf16)
    K, room, launches = args.steps, d["room"], d["launches"]
    ms_per_step, gpu_ms_per_step, tok_s, prefill_s = d["ms_per_step"], d["gpu_ms_per_step"], d["tok_s"], d["prefill_s"]
    tokens, wall, achieved, launch_s = d["tokens"], d["wall"], d["achieved"], d["launch_s"]
    bytes_per_launch, algo_bytes, persistent, kernel = d["bytes_per_launch"], d["algo_bytes"], d["persistent"], d["kernel"]

    info = _lib.pg_device_info()
    _lib.load().pg_device_query(0, C.byref(info))

    result = {
        "metric": (f"decode tokens/sec, GPT-2 {args.model} int8-stored weights bs=1" if args.int8
                   else f"decode tokens/sec, GPT-2 {args.model} bf16-stored weights bs=1" if args.bf16
                   else "decode tokens/sec, GPT-2 XL 1.5B fp32 bs=1" if args.model == "xl"
                   else f"decode tokens/sec, GPT-2 {args.model} fp32 bs=1"),
        "value": round(tok_s, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"GPT-2 {args.model} {'int8-stored weights, fp32 arithmetic,' if args.int8 else 'bf16-stored weights, fp32 arithmetic,' if args.bf16 else 'fp32'} "
                               f"B=1 greedy decode, KV cache prefilled to "
                               f"{n_prefill} tokens, positions {n_prefill}..{n_prefill + min(K, room - 1) - 1}",
                   "weights": "seeded N(0,0.02), biases 0, LayerNorm gamma 1 beta 0",
                   "weight_storage": "int8" if args.int8 else "bf16" if args.bf16 else "f32",
                   "device": info.name.decode() or info.arch.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units,
                   "backend": model.describe()},
        "reference_metric_tokens_per_s": round(tokens / wall, 2),
        "gpu_ms_per_step": round(gpu_ms_per_step, 4),
        "prefill_s": round(prefill_s, 3),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(args, n_prefill, persistent, bytes_per_launch),
                     "traffic_source": TRAFFIC_SOURCE,
                     "kernel": kernel, "launches": launches,
                     "forwards_per_launch": K // launches,
                     "launch_ms": round(launch_s * 1e3, 3),
                     "algorithmic_bytes_per_launch": int(bytes_per_launch),
                     "algorithmic_bytes_per_forward": int(algo_bytes)},
    }

    default_workload = (args.model == "xl" and args.prefill is None and args.decode_path == "auto"
                        and not args.int8 and not args.bf16)
    if default_workload and not args.no_secondary:
        del model
        result["secondary"] = secondary_workloads(cfg, weights)

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, synth.bf16_rounded(weights) if args.bf16 else weights,
                                              ids, n_prefill, args.int8)

    print(json.dumps(result), flush=True)
    return 0


FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X published dense fp32 matrix rate


def measure_decode(model, cfg, ids, n_prefill, steps, warmup, int8=False, bf16=False):
    """Batch-1 greedy decode from a cache prefilled with `ids`: `steps` forwards in passes that
    end at the context limit.  Returns the timings and the HBM roofline figures of the pass."""
    room = cfg.n_positions - n_prefill  # tokens one pass can generate
    cache = model.new_kv_cache()
    t0 = time.time()
    model.prefill(ids, cache)
    prefill_s = time.time() - t0
    log(f"[bench] prefill {n_prefill} tokens: {prefill_s:.2f}s")

    def rewind():
        """Back to the prefilled state with valid logits (one untimed forward)."""
        cache.seq_len = n_prefill - 1
        model.forward_one(int(ids[-1]), cache)

    done = 0
    while done < warmup:
        n = min(warmup - done, room - 1)
        model.decode_greedy(cache, n + 1)
        done += n
        rewind()

    # timed: K forwards in passes of at most room-1 forwards (room tokens)
    steps_left = steps
    wall = gpu = 0.0
    tokens = 0
    kv_total = 0
    launches = 0
    while steps_left > 0:
        n = min(steps_left, room - 1)
        start = cache.seq_len
        toks, st = model.decode_greedy(cache, n + 1)  # n+1 tokens selected, n forwards
        assert len(toks) == n + 1 and cache.seq_len == start + n
        wall += st.decode_time
        gpu += st.gpu_decode_time
        tokens += n + 1
        kv_total += sum(kv_bytes(cfg, p) for p in range(start, start + n))
        steps_left -= n
        launches += 1
        if steps_left > 0:
            rewind()
    K = steps
    # Roofline of the dominant kernel.  On the persistent path one launch of
    # k_decode_persistent<n_embd> runs every forward of a pass (embedding, all blocks,
    # lm_head, argmax); its duration is the HIP-event time the library takes on the
    # launch stream (gpu_decode_time).  Algorithmic bytes: the parameters once per
    # forward plus the K/V rows of positions [0, pos] that forward attends over.
    algo_bytes = weight_bytes(cfg, int8, bf16) + kv_total / K  # per forward
    bytes_per_launch = algo_bytes * K / launches
    launch_s = gpu / launches
    persistent = "decode=persistent" in model.describe()
    kernel = (f"k_decode_persistent<{cfg.n_embd}{', int8 rows' if int8 else ', bf16 rows' if bf16 else ''}>" if persistent
              else "all launches of one decode step (k_gemv dominant)")
    return {"room": room, "launches": launches, "ms_per_step": wall / K * 1e3, "gpu_ms_per_step": gpu / K * 1e3,
            "tok_s": K / wall,  # forwards per second; the reference's tokens/sec adds the free last token
            "prefill_s": prefill_s, "tokens": tokens, "wall": wall,
            "achieved": bytes_per_launch / launch_s / 1e9, "launch_s": launch_s,
            "bytes_per_launch": bytes_per_launch, "algo_bytes": algo_bytes, "persistent": persistent, "kernel": kernel}


def hbm_roofline(achieved_gbs, kernel, traffic=None, traffic_source=None, **extra):
    r = {"bound": "hbm", "achieved": round(achieved_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
         "frac": round(achieved_gbs / HBM_PEAK_GBS, 4), "traffic": traffic, "kernel": kernel, **extra}
    if traffic_source:
        r["traffic_source"] = traffic_source
    return r


def secondary_workloads(xl_cfg, xl_weights):
    """The other configurations of the metric, measured in this same process: small fixed
    step counts, inputs resident, each with the roofline of its own bound."""
    from puppygrad_amd import Gpt2Config, Gpt2HipConfig, Gpt2Model, _lib, synth
    out = {}
    # GPT-2 124M: batch-1 decode of 96 tokens from a 32-token prompt, and the 1024-token prefill
    cfg = Gpt2Config(**synth.GPT2_SMALL)
    w = synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 1)
    model = Gpt2Model.new(cfg, w)
    ids = synth.token_ids(32, synth.TOKEN_SEED_BASE + 1, cfg.vocab_size)
    d = measure_decode(model, cfg, ids, 32, 96, 8)
    out["gpt2_124m_decode_b1"] = {
        "workload": "GPT-2 small 124M fp32 B=1 greedy decode, KV cache prefilled to 32 tokens, positions 32..127",
        "value": round(d["tok_s"], 1), "unit": "tokens/s", "steps": 96, "ms_per_step": round(d["ms_per_step"], 4),
        "gpu_ms_per_step": round(d["gpu_ms_per_step"], 4),
        "reference_metric_tokens_per_s": round(d["tokens"] / d["wall"], 1),
        "roofline": hbm_roofline(d["achieved"], d["kernel"],
                                 traffic=round(TRAFFIC_RATIO_124M * d["algo_bytes"] * 96),
                                 traffic_source=TRAFFIC_SOURCE_124M, launches=d["launches"],
                                 launch_ms=round(d["launch_s"] * 1e3, 3),
                                 algorithmic_bytes_per_forward=int(d["algo_bytes"]))}
    out["gpt2_124m_prefill_32"] = measure_short_prefill(model, cfg, ids, 32, 60, 6)
    out["gpt2_124m_sampled_stream_b1"] = measure_sampled_stream(model, ids, 128)
    ids = synth.token_ids(1024, synth.TOKEN_SEED_BASE + 2, cfg.vocab_size)
    out["gpt2_124m_prefill_1024"] = measure_prefill(model, cfg, ids, 1024, 60, 6)
    del model, w
    # GPT-2 355M: batch-16 decode steps around the mean cache length of configuration 3
    # (128-token prompts + 256 tokens: 129..383 keys, mean 256)
    cfg = Gpt2Config(**synth.GPT2_MEDIUM)
    model = Gpt2Model.new(cfg, synth.random_weights(cfg, synth.WEIGHT_SEED_BASE + 3))
    out["gpt2_355m_decode_b16"] = measure_batch_decode(model, cfg, 16, 220, 64, False,
                                                       traffic_ratio=TRAFFIC_RATIO_355M_B16)
    del model
    # GPT-2 XL with bf16-stored weights: batch-32 decode steps around the mean cache length of
    # configuration 5 (512-token prompts + 512 tokens: 513..1023 keys, mean 768)
    model = Gpt2Model.new(xl_cfg, xl_weights, Gpt2HipConfig(weight_storage=_lib.PG_STORE_BF16))
    out["gpt2_xl_bf16_decode_b32"] = measure_batch_decode(model, xl_cfg, 32, 752, 24, True,
                                                          traffic_ratio=TRAFFIC_RATIO_XL_BF16_B32)
    out["gpt2_xl_bf16_prefill_b32_512"] = measure_batch_prefill_bf16(model, xl_cfg, 32, 512, 3)
    del model
    return out


def measure_sampled_stream(model, ids, n_new, name="GPT-2 124M"):
    """stream_token_ids_with_stats (rust.rs:548-634) with sampled selection: prompt, then n_new
    tokens whose selection (sample_logits, generation.rs:300-362) runs on the device between the
    forwards, no host round trip per token.  Rates are generated tokens over the decode loop's
    wall time, best of three streams; the greedy stream of the same length stands beside them."""
    from puppygrad_amd import TextGenerationConfig

    def rate(**kw):
        best = 0.0
        for _ in range(3):
            _, st = model.stream_token_ids_with_stats(ids, TextGenerationConfig(n_new, seed=7, **kw))
            if st.decode_time > 0:
                best = max(best, st.generated_tokens / st.decode_time)
        return best

    greedy = rate()
    topk = rate(temperature=0.8, top_k=40)
    topp = rate(temperature=0.8, top_p=0.9)
    pen = rate(temperature=0.8, top_k=40, repeat_penalty=1.2)
    return {"workload": f"{name} fp32 B=1 streamed generation of {n_new} tokens from a {len(ids)}-token prompt, "
                        "temperature 0.8 + top_k 40, selection on the device",
            "value": round(topk, 1), "unit": "tokens/s", "steps": n_new,
            "greedy_tokens_per_s": round(greedy, 1),
            "fraction_of_greedy": round(topk / greedy, 3) if greedy > 0 else None,
            "temperature_0.8_top_p_0.9_tokens_per_s": round(topp, 1),
            "temperature_0.8_top_k_40_repeat_penalty_1.2_tokens_per_s": round(pen, 1)}


def measure_short_prefill(model, cfg, ids, T, steps, warmup):
    """First-token latency of a short prompt (BASELINE config 1's 32 tokens): one prefill of T
    tokens into an empty cache.  With so few rows every weight is read once and the flops are
    cheap: the bound is the weights' bytes at the HBM peak."""
    cache = model.new_kv_cache()
    for _ in range(max(1, warmup)):
        model.prefill(ids, cache).argmax()
    t0 = time.time()
    for _ in range(steps):
        lg = model.prefill(ids, cache)
    lg.argmax()
    sec = (time.time() - t0) / steps
    wbytes = weight_bytes(cfg)
    return {"workload": f"GPT-2 124M fp32 B=1 prefill of a {T}-token prompt into an empty KV cache (first-token latency)",
            "value": round(T / sec, 1), "unit": "tokens/s", "steps": steps, "ms_per_step": round(sec * 1e3, 4),
            "roofline": hbm_roofline(wbytes / sec / 1e9,
                                     "whole prefill (k_gemm_rows32, k_attn_prefill64, k_splitk_reduce_ln, lm_head)",
                                     traffic=TRAFFIC_124M_PREFILL_32 if T == 32 else None,
                                     traffic_source=TRAFFIC_SOURCE_124M_PREFILL if T == 32 else None,
                                     algorithmic_bytes_per_step=int(wbytes))}


def measure_prefill(model, cfg, ids, T, steps, warmup):
    """One prefill of T tokens into an empty cache through the full-sequence path, MFMA-bound:
    wall time over `steps` runs for the whole prefill, and one profiled run (HIP events between
    the launches) for the share of the four projections."""
    C_, I, L, V = cfg.n_embd, cfg.n_inner, cfg.n_layer, cfg.vocab_size
    gemm_flops = 2.0 * T * L * (3 * C_ * C_ + C_ * C_ + 2 * C_ * I)
    attn_flops = 4.0 * C_ * (T * (T + 1) / 2) * L
    flops = gemm_flops + attn_flops + 2.0 * V * C_
    cache = model.new_kv_cache()
    for _ in range(max(1, warmup)):
        model.prefill(ids, cache).argmax()
    t0 = time.time()
    for _ in range(steps):
        lg = model.prefill(ids, cache)
    lg.argmax()
    sec = (time.time() - t0) / steps
    _, prof = model.prefill_profiled(ids, cache)
    gemm_s = prof.qkv_projection + prof.attention_projection + prof.mlp_fc_projection + prof.mlp_projection
    whole = flops / sec / 1e12
    gemm = gemm_flops / gemm_s / 1e12 if gemm_s > 0 else 0.0
    attn = attn_flops / prof.attention / 1e12 if prof.attention > 0 else 0.0
    return {"workload": f"GPT-2 124M fp32 B=1 prefill of {T} tokens into an empty KV cache, final-position logits",
            "value": round(T / sec, 1), "unit": "tokens/s", "steps": steps, "ms_per_step": round(sec * 1e3, 4),
            "roofline": {"bound": "mfma", "achieved": round(whole, 2), "peak": FP32_MFMA_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(whole / FP32_MFMA_PEAK_TFLOPS, 4),
                         "traffic": TRAFFIC_124M_PREFILL_1024 if T == 1024 else None,
                         "traffic_source": TRAFFIC_SOURCE_124M_PREFILL if T == 1024 else None,
                         "kernel": "whole prefill (k_gemm, k_attn_prefill64, LayerNorm, split-K reduces, lm_head)",
                         "algorithmic_flops_per_step": int(flops)},
            "gemm_part": {"ms": round(gemm_s * 1e3, 4), "achieved": round(gemm, 2), "unit": "TFLOP/s",
                          "frac": round(gemm / FP32_MFMA_PEAK_TFLOPS, 4), "flops": int(gemm_flops),
                          "how": "HIP events between the launches of one profiled prefill: the four "
                                 "projections of every layer with their split-K reduces and fused LayerNorms"},
            "attention_part": {"ms": round(prof.attention * 1e3, 4), "achieved": round(attn, 2), "unit": "TFLOP/s",
                               "frac": round(attn / FP32_MFMA_PEAK_TFLOPS, 4), "flops": int(attn_flops)}}


def measure_batch_decode(model, cfg, B, n_prefill, steps, bf16, traffic_ratio=None):
    """B sequences prefilled to n_prefill tokens each, then `steps` greedy steps for all of them.
    A step reads every weight once plus the K/V rows of every sequence: HBM-bound."""
    from puppygrad_amd import synth
    steps = min(steps, cfg.n_positions - n_prefill - 1)
    ids = np.stack([synth.token_ids(n_prefill, synth.TOKEN_SEED_BASE + 100 + b, cfg.vocab_size) for b in range(B)])
    cache = model.new_kv_cache(B)
    model.prefill_batch(ids, cache).argmax()
    toks, st = model.decode_greedy_batch(cache, 4)  # warm-up steps
    model.forward_one_batch(toks[-1], cache)        # the forward of the last selected tokens
    start = cache.seq_len
    toks, st = model.decode_greedy_batch(cache, steps + 1)  # steps + 1 tokens per sequence, steps forwards
    n = st.generated_tokens - 1
    sec = st.gpu_decode_time / n
    C_, I, L, V = cfg.n_embd, cfg.n_inner, cfg.n_layer, cfg.vocab_size
    wbytes = (2 if bf16 else 4) * (L * (4 * C_ * C_ + 2 * C_ * I) + V * C_)
    kvb = sum(kv_bytes(cfg, p) for p in range(start, start + n)) / n * B
    achieved = (wbytes + kvb) / sec / 1e9
    return {"workload": f"GPT-2 n_embd={C_} B={B} greedy decode steps, every KV cache at {start}..{start + n - 1} "
                        f"tokens, weights stored as {'bf16' if bf16 else 'f32'}, fp32 arithmetic",
            "value": round(B / sec, 1), "unit": "tokens/s", "steps": n, "ms_per_step": round(sec * 1e3, 4),
            "roofline": hbm_roofline(achieved, "all launches of one batched step",
                                     traffic=round(traffic_ratio * (wbytes + kvb)) if traffic_ratio else None,
                                     traffic_source=TRAFFIC_SOURCE_355M_B16 if traffic_ratio else None,
                                     algorithmic_bytes_per_step=int(wbytes + kvb))}


BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 matrix rate


def prefill_flops(cfg, B, T):
    """(all, projections only) algorithmic flops of B prompts of T tokens."""
    C_, I, L, V = cfg.n_embd, cfg.n_inner, cfg.n_layer, cfg.vocab_size
    gemm_flops = 2.0 * B * T * L * (3 * C_ * C_ + C_ * C_ + 2 * C_ * I)
    attn_flops = 4.0 * B * C_ * (T * (T + 1) / 2) * L
    return gemm_flops + attn_flops + 2.0 * B * V * C_, gemm_flops


def bf16_prefill_roofline(flops, gemm_flops, sec, traffic=None, traffic_source=None):
    """bf16 rows: the projections run on the bf16 matrix cores, every f32 input cut into three
    bf16 parts (exact products, f32 sums): three matrix instructions' worth of work per
    algorithmic product, so a third of the bf16 peak is this form's ceiling."""
    achieved = flops / sec / 1e12
    r = {"bound": "mfma", "achieved": round(achieved, 2), "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
         "frac": round(achieved / BF16_MFMA_PEAK_TFLOPS, 4), "traffic": traffic, "passes": 3,
         "executed": round((2 * gemm_flops + flops) / sec / 1e12, 2),
         "kernel": "whole prefill (k_gemm_b3 on the bf16 matrix cores, k_attn_prefill64 and lm_head in f32)",
         "algorithmic_flops_per_step": int(flops), "gemm_flops_per_step": int(gemm_flops)}
    if traffic_source:
        r["traffic_source"] = traffic_source
    return r


def measure_batch_prefill_bf16(model, cfg, B, T, steps):
    """B prompts of T tokens through the layers at once, weights stored as bf16."""
    from puppygrad_amd import synth
    ids = np.stack([synth.token_ids(T, synth.TOKEN_SEED_BASE + 100 + b, cfg.vocab_size) for b in range(B)])
    cache = model.new_kv_cache(B)
    model.prefill_batch(ids, cache).argmax()
    t0 = time.time()
    for _ in range(steps):
        lg = model.prefill_batch(ids, cache)
    lg.argmax()
    sec = (time.time() - t0) / steps
    flops, gemm_flops = prefill_flops(cfg, B, T)
    return {"workload": f"GPT-2 n_embd={cfg.n_embd} B={B} prefill of {T} tokens each into empty KV caches, "
                        f"weights stored as bf16, f32 inputs and sums",
            "value": round(B * T / sec, 1), "unit": "tokens/s", "steps": steps, "ms_per_step": round(sec * 1e3, 3),
            "roofline": bf16_prefill_roofline(
                flops, gemm_flops, sec,
                traffic=TRAFFIC_XL_BF16_PREFILL_B32_512 if (cfg.n_embd, B, T) == (1600, 32, 512) else None,
                traffic_source=TRAFFIC_SOURCE_XL_BF16_PREFILL if (cfg.n_embd, B, T) == (1600, 32, 512) else None)}


def bench_prefill(args, cfg, model, ids, n_prefill) -> int:
    """Secondary workload (prompt processing, e.g. GPT-2 124M with 1024 tokens): a step is one
    prefill of n_prefill tokens into an empty cache through the GEMM path; with --batch B > 1
    (given explicitly) B prompts of that length at once (pg_gpt2_prefill_batch).  Algorithmic
    flops: the four projections of every layer over all tokens, causal attention
    (QK^T and PV over the lower triangle), and the lm_head row of the last token."""
    from puppygrad_amd import synth
    T = n_prefill
    B = args.batch if args.batch_given else 1
    flops, gemm_flops = prefill_flops(cfg, B, T)
    cache = model.new_kv_cache(B)
    if B > 1:
        ids = np.stack([synth.token_ids(T, synth.TOKEN_SEED_BASE + 100 + b, cfg.vocab_size) for b in range(B)])

    def one():
        if B > 1:
            return model.prefill_batch(ids, cache)
        cache.seq_len = 0
        return model.prefill(ids, cache)

    for _ in range(max(1, args.warmup)):
        one().argmax()
    t0 = time.time()
    for _ in range(args.steps):
        lg = one()
    lg.argmax()  # waits for the last prefill
    wall = time.time() - t0
    sec = wall / args.steps
    info = _devinfo()
    achieved = flops / sec / 1e12
    stored = "bf16-stored weights" if args.bf16 else "fp32"
    result = {
        "metric": f"prefill tokens/sec, GPT-2 {args.model} {stored} bs={B}, {T}-token prompt",
        "value": round(B * T / sec, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": max(1, args.warmup), "ms_per_step": round(sec * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"GPT-2 {args.model} {stored} B={B} prefill of {T} tokens into an empty KV cache",
                   "weights": "seeded N(0,0.02), biases 0, LayerNorm gamma 1 beta 0",
                   "device": info.name.decode() or info.arch.decode(), "compute_units": info.compute_units,
                   "backend": model.describe()},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": FP32_MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "whole prefill (k_gemm, or k_gemm_b9 from 1024 rows on where it is faster; "
                               "k_attn_prefill64, LayerNorm, split-K reduces, lm_head)",
                     "algorithmic_flops_per_step": int(flops), "gemm_flops_per_step": int(gemm_flops)},
    }
    if args.bf16:
        counted = (cfg.n_embd, B, T) == (1600, 32, 512)
        result["roofline"] = bf16_prefill_roofline(
            flops, gemm_flops, sec, traffic=TRAFFIC_XL_BF16_PREFILL_B32_512 if counted else None,
            traffic_source=TRAFFIC_SOURCE_XL_BF16_PREFILL if counted else None)
    # A short prompt reads every weight once for few rows: below about 52 rows the weights'
    # bytes at the HBM peak take longer than the flops at the MFMA peak, and HBM is the bound.
    wbytes = weight_bytes(cfg, bf16=args.bf16)
    if wbytes / (HBM_PEAK_GBS * 1e9) > flops / (FP32_MFMA_PEAK_TFLOPS * 1e12):
        gbs = wbytes / sec / 1e9
        result["roofline"] = hbm_roofline(gbs, "whole prefill (k_gemm_rows32, k_attn_prefill64, reduce + LayerNorm, lm_head)",
                                          algorithmic_bytes_per_step=int(wbytes))
    print(json.dumps(result), flush=True)
    return 0


def bench_batch_decode(args, cfg, model, n_prefill) -> int:
    """Secondary workload (batched decode, e.g. 355M batch 16 or XL bf16 batch 32): --batch sequences
    prefilled to n_prefill tokens each, then --steps greedy steps for all of them.  A step
    reads every weight once plus the K/V rows of every sequence: HBM-bound."""
    from puppygrad_amd import synth
    B = args.batch
    room = cfg.n_positions - n_prefill
    steps = min(args.steps, room - 1)
    ids = np.stack([synth.token_ids(n_prefill, synth.TOKEN_SEED_BASE + 100 + b, cfg.vocab_size) for b in range(B)])
    cache = model.new_kv_cache(B)
    t0 = time.time()
    model.prefill_batch(ids, cache).argmax()
    prefill_s = time.time() - t0
    toks, st = model.decode_greedy_batch(cache, steps + 1)  # steps + 1 tokens per sequence, steps forwards
    n = st.generated_tokens - 1
    sec = st.gpu_decode_time / n
    C_, I, L, V = cfg.n_embd, cfg.n_inner, cfg.n_layer, cfg.vocab_size
    wbytes = (2 if args.bf16 else 4) * (L * (4 * C_ * C_ + 2 * C_ * I) + V * C_)
    kvb = sum(kv_bytes(cfg, p) for p in range(n_prefill, n_prefill + n)) / n * B
    achieved = (wbytes + kvb) / sec / 1e9
    info = _devinfo()
    result = {
        "metric": f"batched decode tokens/sec, GPT-2 {args.model} {'bf16-stored' if args.bf16 else 'fp32'} bs={B}",
        "value": round(B / sec, 1), "unit": "tokens/s", "n_gpus": 1, "steps": n, "warmup": 0,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"GPT-2 {args.model} B={B} greedy decode, every KV cache prefilled to {n_prefill} "
                               f"tokens, weights stored as {'bf16' if args.bf16 else 'f32'}",
                   "device": info.name.decode() or info.arch.decode(), "compute_units": info.compute_units,
                   "backend": model.describe()},
        "prefill_s": round(prefill_s, 3),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "all launches of one batched step",
                     "algorithmic_bytes_per_step": int(wbytes + kvb)},
    }
    print(json.dumps(result), flush=True)
    return 0


def _devinfo():
    from puppygrad_amd import _lib
    info = _lib.pg_device_info()
    _lib.load().pg_device_query(0, C.byref(info))
    return info


# HBM bytes per algorithmic byte of k_decode_persistent<1600> on the headline workload, from
# rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this file, each scaled by what the same
# counter reads for a plain copy kernel of known size
# (profiles/k_decode_persistent_1600_xl_decode_traffic.txt has the counters and the factors).
TRAFFIC_RATIO_XL = 1.0256
TRAFFIC_SOURCE = "profiles/k_decode_persistent_1600_xl_decode_traffic.txt"
# The same for k_decode_persistent<768> on the 124M decode (127 forwards from 32 tokens) and for
# the launches of one 355M batch-16 step (16 steps at 224..239 keys), from runs of this file
# with --model small and with --workload batch-decode.
TRAFFIC_RATIO_124M = 0.983
TRAFFIC_SOURCE_124M = "profiles/k_decode_persistent_768_124m_decode.txt"
# HBM bytes of one 124M prefill (FETCH_SIZE + WRITE_SIZE of all its launches, scaled)
TRAFFIC_124M_PREFILL_1024 = 3208200000
TRAFFIC_124M_PREFILL_32 = 631400000
TRAFFIC_SOURCE_124M_PREFILL = "profiles/prefill_124m_traffic.txt"
TRAFFIC_RATIO_355M_B16 = 1.093
TRAFFIC_RATIO_XL_BF16_B32 = 1.073  # same file, section (c)
TRAFFIC_SOURCE_355M_B16 = "profiles/batched_decode_355m_b16_xl_bf16_b32.txt"
# Bytes through the L2s to and from the fabric per XL bf16 prefill of 32 x 512 tokens (FETCH_SIZE
# scaled by 1.9994 + WRITE_SIZE over all launches of a step; most of the reads are operand
# re-reads that the Infinity Cache serves).
TRAFFIC_XL_BF16_PREFILL_B32_512 = 573030000000
TRAFFIC_SOURCE_XL_BF16_PREFILL = "profiles/k_gemm_b3_xl_bf16_prefill_b32_512.txt"


def measured_traffic(args, n_prefill, persistent, bytes_per_launch):
    """The kernel's HBM traffic per launch: the measured ratio applied to this launch's
    algorithmic bytes (the ratio was taken at 127 forwards per launch; it does not depend on
    their number, every forward streams the same weights)."""
    if args.model == "xl" and n_prefill == 896 and persistent and not args.int8 and not args.bf16:
        return round(TRAFFIC_RATIO_XL * bytes_per_launch)
    return None


def cpu_baseline(cfg, weights, ids, n_prefill, int8=False):
    """The oracle (a C++ restatement of the reference's CPU path, AVX dot and
    round-robin chunked thread pool) timed on this host: a bounded sample of
    forward_one steps at the benchmark's context length."""
    import oracle
    cores = len(os.sched_getaffinity(0))
    threads = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    t0 = time.time()
    q = 1 if int8 else 0  # quantized_weights (src/models/gpt2/options.rs:62)
    ref = oracle.Model(cfg, weights, oracle.rust_config(threads, quantized_weights=q))
    log(f"[bench] cpu oracle build: {time.time() - t0:.1f}s, threads={threads}")
    rcache = ref.new_kv_cache()
    step_ids = [int(ids[i % len(ids)]) for i in range(64)]
    # 1 warmup step, then as many steps as fit in about 15 s (at least 3)
    sec, _ = ref.timed_forward_steps(rcache, n_prefill, step_ids[:1])
    n = int(max(3, min(48, 15.0 / max(sec, 1e-3))))
    runs = []
    for _ in range(3):
        s, _ = ref.timed_forward_steps(rcache, n_prefill, step_ids[:max(1, n // 3)])
        runs.append(max(1, n // 3) / s)
    runs.sort()
    one = oracle.Model(cfg, weights, oracle.rust_config(1, quantized_weights=q))
    c1 = one.new_kv_cache()
    one.timed_forward_steps(c1, n_prefill, step_ids[:1])
    s1, _ = one.timed_forward_steps(c1, n_prefill, step_ids[:3])
    return {"value": round(runs[1], 3), "unit": "tokens/s", "cores": threads, "kind": "port",
            "single_thread_value": round(3 / s1, 3),
            "sample": f"median of 3 runs of {max(1, n // 3)} forward_one steps starting at cache length "
                      f"{n_prefill} (KV values zero-filled; timing does not depend on them), "
                      f"default Gpt2RustConfig thresholds"}


if __name__ == "__main__":
    sys.exit(main())
