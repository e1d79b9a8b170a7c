"""Shared test helpers: an independent float64 GPT-2 in matrix form, fixtures, tolerances."""
from pathlib import Path

import numpy as np

from puppygrad_amd import Gpt2Config, synth

GOLDEN = Path(__file__).resolve().parent / "golden"

# north-star logit tolerance for the fp32 path
ABS_TOL, REL_TOL = 1e-4, 1e-3


def assert_logits_close(got, want, abs_tol=ABS_TOL, rel_tol=REL_TOL, what="logits"):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = np.abs(got - want)
    bound = abs_tol + rel_tol * np.abs(want)
    bad = err > bound
    assert not bad.any(), (f"{what}: {bad.sum()} of {bad.size} outside {abs_tol} abs + {rel_tol} "
                           f"rel; max err {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}")


def numpy_gpt2_forward(cfg: Gpt2Config, w, ids, lm_head=None) -> np.ndarray:
    """GPT-2 in float64 with whole-matrix numpy ops on the HF [in,out] weights.
    Written from the architecture, not from the oracle's loops: a transposed
    weight, a wrong head slice or a dropped residual fails against it.
    lm_head ([vocab, n_embd]) replaces the tied wte in the final projection only."""
    f = lambda a, *s: np.asarray(a, np.float64).reshape(*s)
    C, H, I, V = cfg.n_embd, cfg.n_head, cfg.n_inner, cfg.vocab_size
    hd = C // H
    T = len(ids)
    wte, wpe = f(w.wte, V, C), f(w.wpe, cfg.n_positions, C)
    x = wte[np.asarray(ids)] + wpe[:T]

    def ln(v, g, b):
        mu = v.mean(-1, keepdims=True)
        var = ((v - mu) ** 2).mean(-1, keepdims=True)
        return (v - mu) / np.sqrt(var + cfg.layer_norm_epsilon) * f(g, C) + f(b, C)

    mask = np.tril(np.ones((T, T), bool))
    for b in w.blocks:
        qkv = ln(x, b.ln_1_g, b.ln_1_b) @ f(b.c_attn_w, C, 3 * C) + f(b.c_attn_b, 3 * C)
        q, k, v = [qkv[:, i * C:(i + 1) * C].reshape(T, H, hd).transpose(1, 0, 2) for i in range(3)]
        s = q @ k.transpose(0, 2, 1) / np.sqrt(hd)
        s = np.where(mask, s, -np.inf)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        a = (p @ v).transpose(1, 0, 2).reshape(T, C)
        x = x + a @ f(b.c_proj_w, C, C) + f(b.c_proj_b, C)
        h = ln(x, b.ln_2_g, b.ln_2_b) @ f(b.c_fc_w, C, I) + f(b.c_fc_b, I)
        h = 0.5 * h * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (h + 0.044715 * h ** 3)))
        x = x + h @ f(b.c_proj_mlp_w, I, C) + f(b.c_proj_mlp_b, C)
    head = wte if lm_head is None else f(lm_head, V, C)
    return ln(x, w.ln_f_g, w.ln_f_b) @ head.T


def load_golden(name: str):
    z = np.load(GOLDEN / f"{name}.npz")
    c = [int(v) for v in z["config"]]
    cfg = Gpt2Config(vocab_size=c[0], n_positions=c[1], n_embd=c[2], n_layer=c[3], n_head=c[4],
                     n_inner=c[5], layer_norm_epsilon=float(z["eps"]))
    w = synth.random_weights(cfg, int(z["weight_seed"]), perturb=bool(z["perturb"]))
    return cfg, w, z


def small_cases():
    """(name, config, weights, ids) for models small enough for any test."""
    out = []
    cfg = synth.tiny_config()
    out.append(("tiny", cfg, synth.tiny_weights(cfg), [1, 2, 3]))
    cfg = Gpt2Config(vocab_size=131, n_positions=40, n_embd=128, n_layer=2, n_head=2)
    out.append(("c128", cfg, synth.random_weights(cfg, 0x5EED0201, perturb=True),
                list(synth.token_ids(17, 0x70C00201, 131))))
    cfg = Gpt2Config(vocab_size=300, n_positions=64, n_embd=36, n_layer=2, n_head=3, n_inner=100)
    out.append(("odd", cfg, synth.random_weights(cfg, 0x5EED0202, std=0.08, perturb=True),
                list(synth.token_ids(23, 0x70C00202, 300))))
    return out


class DeviceArray:
    """A host array mirrored in a device buffer of the library (pg_device_*)."""

    def __init__(self, host, dtype=np.float32):
        import ctypes as C
        from puppygrad_amd import _lib
        self._C, self.lib = C, _lib.load()
        self.host = np.ascontiguousarray(host, dtype=dtype)
        self.ptr = C.c_void_p()
        assert self.lib.pg_device_alloc(0, self.host.nbytes, C.byref(self.ptr)) == 0
        assert self.lib.pg_device_upload(0, self.ptr, self.host.ctypes.data_as(C.c_void_p),
                                         self.host.nbytes) == 0

    def download(self) -> np.ndarray:
        out = np.empty_like(self.host)
        assert self.lib.pg_device_download(0, out.ctypes.data_as(self._C.c_void_p), self.ptr,
                                           out.nbytes) == 0
        return out

    def free(self):
        assert self.lib.pg_device_free(0, self.ptr) == 0
