"""Per-hop breakdown of the persistent decode kernel (k_decode_persistent) from the timestamps
a development build of the library takes inside the kernel.

    python -m puppygrad_amd.build --stamps
    python -m puppygrad_amd.decode_stamps small|medium|xl [n_prefill] [n_tokens]

The build compiles the library with PG_DECODE_PROF_BUILD (libpuppygrad_hip_stamps.so); a launch
then keeps, for its last token, the shader clock (s_memtime) of every phase of every layer in LDS
and writes them out per workgroup, with two readings of the 100 MHz wall clock, to the file named
by PG_DECODE_PROF.  The shader clocks of different XCDs are not synchronised, so every workgroup's
stamps are converted to the wall clock with its own rate and offset before they are compared."""
import os
import sys
import tempfile

import numpy as np

from . import build as _build


def main(argv):
    os.environ.setdefault("PUPPYGRAD_HIP_LIB", str(_build.STAMPS_LIB_PATH))
    # (a caller may name the file of raw stamps itself, to keep it)
    out = os.environ.setdefault("PG_DECODE_PROF", os.path.join(tempfile.gettempdir(), "pg_decode_stamps.bin"))
    from . import Gpt2Config, Gpt2Model, synth  # after the environment is set: the library loads on import
    name = argv[1] if len(argv) > 1 else 'small'
    kw = {'xl': synth.GPT2_XL, 'small': synth.GPT2_SMALL, 'medium': synth.GPT2_MEDIUM}[name]
    cfg = Gpt2Config(**kw)
    npre = int(argv[2]) if len(argv) > 2 else {'xl': 896, 'small': 32, 'medium': 128}[name]
    ntok = int(argv[3]) if len(argv) > 3 else 33
    w = synth.random_weights(cfg, 1)
    ids = synth.token_ids(npre, 2, cfg.vocab_size)
    m = Gpt2Model.new(cfg, w)
    c = m.new_kv_cache()
    m.prefill(ids, c)
    toks, st = m.decode_greedy(c, ntok)
    print(name, 'decode', st.gpu_decode_time / (ntok - 1) * 1e3, 'ms/token (with stamps)')
    L = cfg.n_layer
    raw = np.fromfile(out, dtype=np.uint64).reshape(-1, L + 1, 16).astype(np.float64)
    G = raw.shape[0]
    # per-WG conversion of shader-clock stamps to the global 100 MHz wall clock
    S0, W0, W1, S1 = raw[:, L, 7], raw[:, L, 13], raw[:, L, 14], raw[:, L, 15]
    rate = (S1 - S0) / (W1 - W0)   # shader ticks per wall tick
    print('shader clock: %.1f MHz (min %.1f max %.1f)' % (rate.mean() * 100, rate.min() * 100, rate.max() * 100))
    a = np.where(raw > 0, (W0[:, None, None] + (raw - S0[:, None, None]) / rate[:, None, None]) * 0.01, 0.0)
    a[:, L, 13] = W0 * 0.01; a[:, L, 14] = W1 * 0.01
    t_origin = a[:, L, 7][a[:, L, 7] > 0].min()
    a = np.where(a > 0, a - t_origin + 1.0, 0.0)
    def col(l, k):
        v = a[:, l, k]
        return v[v > 0]

    rows = []
    for l in range(1, L):
        F_prev = col(l - 1, 7).max()          # last F store of the previous layer (streamer 0 of each WG)
        A_flag = col(l, 0)                    # service: xsA staged, flag raised
        A_store = col(l, 5)                   # streamer 0: A rows published
        B_done = col(l, 1)                    # service: attention items done (partials / attn published)
        D_flag = col(l, 2)
        D_store = col(l, 11)
        E_flag = col(l, 3)
        E_store = col(l, 6)
        F_flag = col(l, 4)
        F_store = col(l, 7)
        rows.append([A_flag.max() - F_prev, A_store.max() - A_flag.max(), B_done.max() - A_store.max(),
                     D_flag.max() - B_done.max(), D_store.max() - D_flag.max(), E_flag.max() - D_store.max(),
                     E_store.max() - E_flag.max(), F_flag.max() - E_store.max(), F_store.max() - F_flag.max(),
                     F_store.max() - F_prev,
                     A_flag.max() - A_flag.min(), D_flag.max() - D_flag.min(), E_flag.max() - E_flag.min(), F_flag.max() - F_flag.min(),
                     A_flag.min() - F_prev, E_flag.min() - D_store.max(), F_flag.min() - E_store.max(), D_flag.min() - B_done.max()])
    r = np.array(rows)
    names = ['F store->A flag (hop)', 'A flag->A store (product)', 'A store->B done (hop+attn)', 'B done->D flag (hop[+merge])',
             'D flag->D store (product)', 'D store->E flag (hop)', 'E flag->E store (product)', 'E store->F flag (hop)',
             'F flag->F store (product)', 'LAYER', 'spread A flag', 'spread D flag', 'spread E flag', 'spread F flag',
             'last F store->FIRST A flag', 'last D store->FIRST E flag', 'last E store->FIRST F flag', 'last B done->FIRST D flag']
    for n_, v in zip(names, r.T):
        print(f'{n_:32s} mean {v.mean():6.2f}  min {v.min():6.2f}  max {v.max():6.2f}')
    print('token span', a[:, L, 6].max() - a[:, L, 7][a[:, L, 7] > 0].min())


if __name__ == "__main__":
    main(sys.argv)
