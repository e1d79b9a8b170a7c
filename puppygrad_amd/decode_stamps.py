"""Per-hop breakdown of the persistent decode kernel (k_decode_persistent) from the timestamps
a development build of the library takes inside the kernel.

    python -m puppygrad_amd.build --stamps
    python -m puppygrad_amd.decode_stamps small|medium|xl [n_prefill] [n_tokens]
    python -m puppygrad_amd.decode_stamps --read <file of raw stamps> <n_layer>

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


def analyse(path, L, show=print):
    """Prints the per-hop table from a file of raw stamps ([workgroup][L + 1][16] u64)."""
    raw = np.fromfile(path, dtype=np.uint64).reshape(-1, L + 1, 16).astype(np.float64)
    # per-workgroup conversion of shader-clock stamps to the 100 MHz wall clock
    S0, W0, W1, S1 = raw[:, L, 7], raw[:, L, 13], raw[:, L, 14], raw[:, L, 15]
    rate = (S1 - S0) / (W1 - W0)   # shader ticks per wall tick
    show('shader clock: %.1f MHz (min %.1f max %.1f)' % (rate.mean() * 100, rate.min() * 100, rate.max() * 100))
    a = np.where(raw > 0, (W0[:, None, None] + (raw - S0[:, None, None]) / rate[:, None, None]) * 0.01, 0.0)
    # The wall clocks of the eight XCDs are offset against each other by up to a few microseconds
    # (the same amounts at every event of a run, other amounts in the next run).  Workgroup g runs
    # on XCD g % 8: each XCD's mean deviation from the all-workgroup mean over the events of
    # layers 1.. is taken as its offset and removed, so that "first" and "last workgroup" compare
    # times and not clocks.
    events = [0, 5, 2, 11, 3, 6, 4, 7]
    dev = np.zeros(a.shape[0])
    for k in events:
        v = a[:, 1:L, k]
        dev += (v - v.mean(axis=0, keepdims=True)).mean(axis=1)
    dev /= len(events)
    off = np.array([dev[x::8].mean() for x in range(8)])
    show('clock offsets of the XCDs removed (us): ' + ' '.join('%+.2f' % o for o in off))
    b = a.copy()
    for x in range(8):
        b[x::8] -= off[x]
    a = np.where(a > 0, b, 0.0)

    def col(l, k):
        v = a[:, l, k]
        return v[v > 0]

    rows = []
    for l in range(1, L):
        F_prev = col(l - 1, 7).max()          # last F store of the previous layer (streamer 0 of each WG)
        A_flag = col(l, 0)                    # service: xsA staged, flag raised, statistics published
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
        show(f'{n_:32s} mean {v.mean():6.2f}  min {v.min():6.2f}  max {v.max():6.2f}')
    # one workgroup's own clock: the pieces of the c_fc hand-over
    d = lambda k1, k0: raw[:, 1:L, k1] - raw[:, 1:L, k0]
    us = lambda v: (v / rate[:, None] * 0.01)
    if (raw[:, 1:L, 14] > 0).all() and (raw[:, 1:L, 15] > 0).all():
        show('c_fc input, per workgroup: probe round trip %.2f, probe ok -> vector read back %.2f, -> statistics published %.2f'
             % (us(d(13, 14)).mean(), us(d(15, 13)).mean(), us(d(3, 15)).mean()))
    show('tail: last F store -> final input staged %.2f, -> argmax published %.2f (lm_head); token start -> first input staged %.2f'
         % (us(raw[:, L, 5] - raw[:, L - 1, 7]).mean(), us(raw[:, L, 6] - raw[:, L, 5]).mean(),
            us(raw[:, 0, 0] - raw[:, L, 7]).mean()))


def main(argv):
    if len(argv) > 3 and argv[1] == '--read':  # a file of raw stamps kept from an earlier run
        analyse(argv[2], int(argv[3]))
        return
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
    analyse(out, cfg.n_layer)


if __name__ == "__main__":
    main(sys.argv)
