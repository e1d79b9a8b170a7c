"""Seeded synthetic GPT-2 weights and token ids, shared by tests and bench.

Weights are N(0, std) from the reference's splitmix64 (src/models/generation.rs:244-267)
through Box-Muller, generated inside libpuppygrad_hip.so (pg_synth_normal_f32).
One stream per seed; tensors take consecutive ranges of it in this order:
wte, wpe, then per layer c_attn_w, c_proj_w, c_fc_w, c_proj_mlp_w, all in the HF
[in,out] layout.  LayerNorm gamma = 1, beta = 0 and linear biases = 0 unless
`perturb` is set, in which case they get small seeded values so that tests cover
those terms.
"""
from __future__ import annotations

import numpy as np

from . import _lib
from .gpt2 import Gpt2BlockWeights, Gpt2Config, Gpt2Weights

GPT2_SMALL = dict(vocab_size=50257, n_positions=1024, n_embd=768, n_layer=12, n_head=12)
GPT2_MEDIUM = dict(vocab_size=50257, n_positions=1024, n_embd=1024, n_layer=24, n_head=16)
GPT2_LARGE = dict(vocab_size=50257, n_positions=1024, n_embd=1280, n_layer=36, n_head=20)
GPT2_XL = dict(vocab_size=50257, n_positions=1024, n_embd=1600, n_layer=48, n_head=25)

WEIGHT_SEED_BASE = 0x5EED_0000
TOKEN_SEED_BASE = 0x70C0_0000


def normal_f32(n: int, seed: int, first: int, std: float = 0.02) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    _lib.load().pg_synth_normal_f32(_lib.f32p(out), n, seed, first, std)
    return out


def token_ids(n: int, seed: int, vocab: int) -> np.ndarray:
    out = np.empty(n, dtype=np.uint32)
    _lib.load().pg_synth_token_ids(_lib.u32p(out), n, seed, vocab)
    return out


def random_weights(cfg: Gpt2Config, seed: int, std: float = 0.02,
                   perturb: bool = False) -> Gpt2Weights:
    C, I = cfg.n_embd, cfg.n_inner
    pos = 0

    def take(n):
        nonlocal pos
        a = normal_f32(n, seed, pos, std)
        pos += n
        return a

    wte = take(cfg.vocab_size * C)
    wpe = take(cfg.n_positions * C)
    blocks = []
    for _ in range(cfg.n_layer):
        c_attn_w = take(C * 3 * C)
        c_proj_w = take(C * C)
        c_fc_w = take(C * I)
        c_proj_mlp_w = take(I * C)
        blocks.append(Gpt2BlockWeights(
            ln_1_g=np.ones(C, np.float32), ln_1_b=np.zeros(C, np.float32),
            c_attn_w=c_attn_w, c_attn_b=np.zeros(3 * C, np.float32),
            c_proj_w=c_proj_w, c_proj_b=np.zeros(C, np.float32),
            ln_2_g=np.ones(C, np.float32), ln_2_b=np.zeros(C, np.float32),
            c_fc_w=c_fc_w, c_fc_b=np.zeros(I, np.float32),
            c_proj_mlp_w=c_proj_mlp_w, c_proj_mlp_b=np.zeros(C, np.float32)))
    w = Gpt2Weights(wte, wpe, blocks, np.ones(C, np.float32), np.zeros(C, np.float32))
    if perturb:
        # A second stream (seed + 1) for the terms the default init leaves at 0 / 1.
        p = 0

        def small(n, centre):
            nonlocal p
            a = normal_f32(n, seed + 1, p, 0.1) + np.float32(centre)
            p += n
            return a.astype(np.float32)

        for b in w.blocks:
            b.ln_1_g, b.ln_1_b = small(C, 1.0), small(C, 0.0)
            b.c_attn_b, b.c_proj_b = small(3 * C, 0.0), small(C, 0.0)
            b.ln_2_g, b.ln_2_b = small(C, 1.0), small(C, 0.0)
            b.c_fc_b, b.c_proj_mlp_b = small(I, 0.0), small(C, 0.0)
        w.ln_f_g, w.ln_f_b = small(C, 1.0), small(C, 0.0)
    return w


def patterned(n: int, scale: float) -> np.ndarray:
    """The reference's test pattern (src/models/gpt2/rust.rs:2117-2121)."""
    i = np.arange(n, dtype=np.int64)
    return (((i * 17 + 11) % 23).astype(np.float32) - np.float32(11.0)) * np.float32(scale)


def tiny_config() -> Gpt2Config:
    """tiny_config (src/models/gpt2/rust.rs:2082-2092)."""
    return Gpt2Config(vocab_size=8, n_positions=5, n_embd=4, n_layer=1, n_head=2, n_inner=8,
                      layer_norm_epsilon=1e-5)


def tiny_weights(cfg: Gpt2Config) -> Gpt2Weights:
    """tiny_weights (src/models/gpt2/rust.rs:2094-2115)."""
    C, I = cfg.n_embd, cfg.n_inner
    one, zero = (lambda n: np.ones(n, np.float32)), (lambda n: np.zeros(n, np.float32))
    return Gpt2Weights(
        wte=patterned(cfg.vocab_size * C, 0.03), wpe=patterned(cfg.n_positions * C, 0.02),
        blocks=[Gpt2BlockWeights(
            ln_1_g=one(C), ln_1_b=zero(C), c_attn_w=patterned(C * 3 * C, 0.01),
            c_attn_b=zero(3 * C), c_proj_w=patterned(C * C, 0.015), c_proj_b=zero(C),
            ln_2_g=one(C), ln_2_b=zero(C), c_fc_w=patterned(C * I, 0.01), c_fc_b=zero(I),
            c_proj_mlp_w=patterned(I * C, 0.012), c_proj_mlp_b=zero(C))],
        ln_f_g=one(C), ln_f_b=zero(C))


def round_bf16(a: np.ndarray) -> np.ndarray:
    """f32 -> bf16 (round to nearest even) -> f32, as the bf16 weight storage does."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    return r.view(np.float32)


def bf16_rounded(w: Gpt2Weights) -> Gpt2Weights:
    """The weights a bf16-storage model really multiplies with: wte and the four block
    matrices rounded to bf16; LayerNorm parameters, biases and wpe untouched."""
    blocks = [Gpt2BlockWeights(
        ln_1_g=b.ln_1_g, ln_1_b=b.ln_1_b, c_attn_w=round_bf16(b.c_attn_w), c_attn_b=b.c_attn_b,
        c_proj_w=round_bf16(b.c_proj_w), c_proj_b=b.c_proj_b, ln_2_g=b.ln_2_g, ln_2_b=b.ln_2_b,
        c_fc_w=round_bf16(b.c_fc_w), c_fc_b=b.c_fc_b, c_proj_mlp_w=round_bf16(b.c_proj_mlp_w),
        c_proj_mlp_b=b.c_proj_mlp_b) for b in w.blocks]
    return Gpt2Weights(wte=round_bf16(w.wte), wpe=w.wpe, blocks=blocks, ln_f_g=w.ln_f_g,
                       ln_f_b=w.ln_f_b)
