"""Writes tests/golden/hf_*.npz: logits of a locally constructed Hugging Face
GPT2LMHeadModel (float64, eager attention, gelu_new) on this repo's seeded
synthetic weights.  HF GPT-2 is an independent implementation of the same
architecture (Conv1D [in,out] weights, pre-LN, tied lm_head, 1/sqrt(head_dim)),
so these vectors pin the oracle's full model without running the reference.

Run from the repo root:  python tests/golden/make_hf_golden.py
Needs: torch, transformers (no network), and the built libpuppygrad_hip.so for
the weight generator (CPU only).
"""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from puppygrad_amd import Gpt2Config, synth  # noqa: E402

OUT = Path(__file__).resolve().parent

CASES = {
    # name: (config kwargs, weight seed, perturb, n prompt ids, token seed)
    "hf_c128_l2": (dict(vocab_size=97, n_positions=32, n_embd=128, n_layer=2, n_head=2), 0x5EED0101,
                   True, 12, 0x70C00101),
    "hf_c192_l3_h3": (dict(vocab_size=211, n_positions=48, n_embd=192, n_layer=3, n_head=3),
                      0x5EED0102, True, 40, 0x70C00102),
    "hf_gpt2_small": (synth.GPT2_SMALL, 0x5EED0001, False, 16, 0x70C00001),
}


def hf_logits(cfg: Gpt2Config, w, ids: np.ndarray) -> np.ndarray:
    from transformers import GPT2Config, GPT2LMHeadModel
    hc = GPT2Config(vocab_size=cfg.vocab_size, n_positions=cfg.n_positions, n_embd=cfg.n_embd,
                    n_layer=cfg.n_layer, n_head=cfg.n_head, n_inner=cfg.n_inner,
                    activation_function="gelu_new", layer_norm_epsilon=cfg.layer_norm_epsilon,
                    resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0, bos_token_id=0,
                    eos_token_id=0, attn_implementation="eager")
    m = GPT2LMHeadModel(hc).double().eval()
    C, I = cfg.n_embd, cfg.n_inner
    t = lambda a, *shape: torch.from_numpy(np.asarray(a, np.float64).reshape(*shape))
    sd = {"transformer.wte.weight": t(w.wte, cfg.vocab_size, C),
          "transformer.wpe.weight": t(w.wpe, cfg.n_positions, C),
          "transformer.ln_f.weight": t(w.ln_f_g, C), "transformer.ln_f.bias": t(w.ln_f_b, C),
          "lm_head.weight": t(w.wte, cfg.vocab_size, C)}
    for i, b in enumerate(w.blocks):
        p = f"transformer.h.{i}."
        sd.update({p + "ln_1.weight": t(b.ln_1_g, C), p + "ln_1.bias": t(b.ln_1_b, C),
                   p + "attn.c_attn.weight": t(b.c_attn_w, C, 3 * C),
                   p + "attn.c_attn.bias": t(b.c_attn_b, 3 * C),
                   p + "attn.c_proj.weight": t(b.c_proj_w, C, C),
                   p + "attn.c_proj.bias": t(b.c_proj_b, C),
                   p + "ln_2.weight": t(b.ln_2_g, C), p + "ln_2.bias": t(b.ln_2_b, C),
                   p + "mlp.c_fc.weight": t(b.c_fc_w, C, I), p + "mlp.c_fc.bias": t(b.c_fc_b, I),
                   p + "mlp.c_proj.weight": t(b.c_proj_mlp_w, I, C),
                   p + "mlp.c_proj.bias": t(b.c_proj_mlp_b, C)})
    missing, unexpected = m.load_state_dict(sd, strict=False)
    missing = [k for k in missing if not k.endswith(".attn.bias") and not k.endswith("masked_bias")]
    assert not missing and not unexpected, (missing, unexpected)
    with torch.no_grad():
        out = m(torch.from_numpy(ids.astype(np.int64))[None]).logits[0]
    return out.numpy()


def main():
    for name, (ckw, wseed, perturb, n, tseed) in CASES.items():
        cfg = Gpt2Config(**ckw)
        w = synth.random_weights(cfg, wseed, perturb=perturb)
        ids = synth.token_ids(n, tseed, cfg.vocab_size)
        logits = hf_logits(cfg, w, ids)  # [n][V] float64
        if cfg.vocab_size > 1000:
            # keep the file small: last position only, every 53rd id plus the top 32
            last = logits[-1]
            cols = np.unique(np.concatenate([np.arange(0, cfg.vocab_size, 53),
                                             np.argsort(-last)[:32]])).astype(np.int64)
            rows = np.array([n - 1], np.int64)
            vals = last[cols][None].astype(np.float32)
            top = np.argsort(-last)[:2]
            extra = dict(argmax=np.int64(top[0]), top2_gap=np.float64(last[top[0]] - last[top[1]]))
        else:
            cols = np.arange(cfg.vocab_size, dtype=np.int64)
            rows = np.arange(n, dtype=np.int64)
            vals = logits.astype(np.float32)
            extra = {}
        np.savez_compressed(OUT / f"{name}.npz", config=np.array(
            [cfg.vocab_size, cfg.n_positions, cfg.n_embd, cfg.n_layer, cfg.n_head, cfg.n_inner],
            np.int64), eps=np.float64(cfg.layer_norm_epsilon), weight_seed=np.uint64(wseed),
            perturb=np.bool_(perturb), token_seed=np.uint64(tseed), ids=ids, rows=rows, cols=cols,
            logits=vals, **extra)
        print(name, vals.shape, float(np.abs(vals).max()))


if __name__ == "__main__":
    main()
