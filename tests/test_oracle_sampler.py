"""Pins the oracle's generation.rs restatement: the reference's known-answer
tests (src/models/generation.rs:368-403), splitmix64 integer known answers, and
brute force on small inputs."""
import math

import numpy as np
import pytest

import oracle

MASK = (1 << 64) - 1


def splitmix64_closed_form(seed, n):
    """The integer recurrence of SmallRng written out (generation.rs:250-261)."""
    state = seed ^ 0x9E3779B97F4A7C15
    out = []
    for _ in range(n):
        state = (state + 0x9E3779B97F4A7C15) & MASK
        v = state
        v = ((v ^ (v >> 30)) * 0xBF58476D1CE4E5B9) & MASK
        v = ((v ^ (v >> 27)) * 0x94D049BB133111EB) & MASK
        out.append(v ^ (v >> 31))
    return out


def test_splitmix64_known_answers():
    r = oracle.SmallRng(299792458)
    got = [r.next_u64() for _ in range(3)]
    assert got == [0x2788DF83E85DDB82, 0x8D4AF85AB3C903F9, 0xE889F1995D0FFA75]
    assert got == splitmix64_closed_form(299792458, 3)
    assert oracle.SmallRng(0).next_u64() == 0x6E789E6AA1B965F4
    r = oracle.SmallRng(299792458)
    u = [r.next_unit_f64() for _ in range(3)]
    assert u == [0.1544322678604354, 0.5519252034608009, 0.9083548545286816]
    assert all(0.0 <= x < 1.0 for x in u)


def test_repeat_penalty_can_change_greedy_selection():
    # generation.rs:372-383
    s = oracle.LogitsSampler(299792458)
    assert s.select_next_token([1.0, 3.0, 2.0], [1], oracle.sampling(repeat_penalty=2.0)) == 2


def test_top_k_one_samples_best_candidate():
    # generation.rs:385-396
    s = oracle.LogitsSampler(299792458)
    assert s.select_next_token([0.0, 10.0, 9.0], [], oracle.sampling(temperature=1.0, top_k=1)) == 1


def test_validates_sampling_config():
    # generation.rs:398-403 and the other branches of validate (91-117)
    with pytest.raises(oracle.OracleError, match="top_p"):
        oracle.validate_generation(oracle.sampling(top_p=2.0))
    with pytest.raises(oracle.OracleError, match="top_k"):
        c = oracle.sampling()
        c.has_top_k, c.top_k = 1, 0
        oracle.validate_generation(c)
    with pytest.raises(oracle.OracleError, match="temperature"):
        oracle.validate_generation(oracle.sampling(temperature=-1.0))
    with pytest.raises(oracle.OracleError, match="repeat_penalty"):
        oracle.validate_generation(oracle.sampling(repeat_penalty=0.0))
    oracle.validate_generation(oracle.sampling(temperature=0.7, top_p=1.0, top_k=5))


def test_argmax_tie_and_nan_rules():
    inf, nan = float("inf"), float("nan")
    assert oracle.argmax_logits([1.0, 3.0, 3.0, 2.0]) == 1      # first maximum wins
    assert oracle.argmax_logits([-inf, -inf]) == 0               # nothing beats -inf
    assert oracle.argmax_logits([nan, nan, nan]) == 0
    assert oracle.argmax_logits([1.0, nan, 0.5]) == 0            # NaN never selected
    assert oracle.argmax_logits([nan, 1.0, inf, inf]) == 2
    assert oracle.argmax_logits([-5.0]) == 0


def test_repeat_penalty_rules():
    # negatives are multiplied, others divided; ids counted once; window is the last n
    cfg = oracle.sampling(repeat_penalty=2.0, repeat_last_n=2)
    s = oracle.LogitsSampler(1)
    # history [0,1,2]: window = last two ids {2,1}; id 0 is untouched and wins
    assert s.select_next_token([2.1, 4.0, 4.0], [0, 1, 2], cfg) == 0
    # negative logit gets more negative: [-1,-0.9] with id 1 penalised -> -1.8
    assert s.select_next_token([-1.0, -0.9], [1], cfg) == 0
    # duplicate ids penalised once: 4/2 = 2 > 1.5
    assert s.select_next_token([1.5, 4.0], [1, 1], cfg) == 1
    # out-of-range history ids are ignored
    assert s.select_next_token([1.0, 2.0], [7], cfg) == 1
    # last_n = 0 disables
    assert s.select_next_token([1.0, 1.5], [1], oracle.sampling(repeat_penalty=9.0, repeat_last_n=0)) == 1


def brute_force_sample(logits, temperature, top_k, top_p, u):
    """Direct statement of the sampling rule on a short list (python floats are f64)."""
    cand = [(i, float(np.float32(l))) for i, l in enumerate(logits) if math.isfinite(l)]
    cand.sort(key=lambda t: -t[1])  # python's sort is stable
    if top_k is not None:
        cand = cand[:top_k]
    T = float(np.float32(temperature))
    mx = cand[0][1] / T
    w = [(i, math.exp(l / T - mx)) for i, l in cand]
    if top_p is not None:
        full = sum(x for _, x in w)
        cum, keep = 0.0, 0
        for _, x in w:
            cum += x
            keep += 1
            if cum / full >= float(np.float32(top_p)):
                break
        w = w[:max(keep, 1)]
    target = u * sum(x for _, x in w)
    for i, x in w:
        target -= x
        if target <= 0.0:
            return i
    return w[-1][0]


@pytest.mark.parametrize("top_k,top_p", [(None, None), (3, None), (None, 0.6), (2, 0.9), (5, 0.05)])
def test_sampler_against_brute_force(top_k, top_p):
    logits = [0.3, 2.0, -1.0, 1.9, float("-inf")]
    for seed in range(40):
        s = oracle.LogitsSampler(seed)
        u = oracle.SmallRng(seed).next_unit_f64()
        got = s.select_next_token(logits, [], oracle.sampling(temperature=0.8, top_k=top_k, top_p=top_p))
        assert got == brute_force_sample(logits, 0.8, top_k, top_p, u)


def test_sampler_stable_order_on_ties_and_all_nonfinite():
    # equal logits keep index order under the stable sort, so top_k=1 picks the first
    s = oracle.LogitsSampler(3)
    assert s.select_next_token([1.0, 1.0, 1.0], [], oracle.sampling(temperature=1.0, top_k=1)) == 0
    with pytest.raises(oracle.OracleError, match="non-finite"):
        s.select_next_token([float("nan"), float("inf")], [], oracle.sampling(temperature=1.0))


def test_sampling_frequencies_follow_softmax():
    logits = np.array([0.0, 1.0, 2.0], np.float32)
    p = np.exp(logits - logits.max()); p /= p.sum()
    s = oracle.LogitsSampler(12345)
    cfg = oracle.sampling(temperature=1.0)
    counts = np.bincount([s.select_next_token(logits, [], cfg) for _ in range(6000)], minlength=3)
    np.testing.assert_allclose(counts / 6000.0, p, atol=0.02)
