"""HIP kernels against the oracle, op by op, through the C ABI (pg_op_*)."""
import ctypes as C

import numpy as np
import pytest

import oracle
from puppygrad_amd import _lib
from puppygrad_amd.synth import patterned

pytestmark = pytest.mark.gpu


def L():
    return _lib.load()


def ok(status):
    assert status == 0, L().pg_last_error_message().decode()


def hip_dense(x, rows, k, n, w, b):
    out = np.empty(rows * n, np.float32)
    ok(L().pg_op_dense(0, _lib.f32p(x), rows, k, n, _lib.f32p(w), _lib.f32p(b), _lib.f32p(out)))
    return out


@pytest.mark.parametrize("rows,k,n", [(1, 768, 2304), (1, 768, 768), (1, 3072, 768), (1, 1600, 4800),
                                      (1, 6400, 1600), (2, 1024, 4096), (1, 4, 12), (3, 37, 5),
                                      (1, 100, 1), (1, 1600, 50257), (1, 8, 4)])
def test_dense_matches_oracle(rows, k, n):
    rng = np.random.default_rng(k * 31 + n)
    x = rng.standard_normal(rows * k).astype(np.float32)
    w = (rng.standard_normal(n * k) * 0.02).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    got = hip_dense(x, rows, k, n, w, b)
    want = oracle.transposed_dense(x, rows, k, n, w, b)
    np.testing.assert_allclose(got, want, atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("rows,k,n", [(16, 768, 2304), (1024, 768, 768), (100, 3072, 768), (128, 1600, 4800),
                                      (37, 64, 50), (1000, 1024, 4096), (33, 16, 129), (64, 6400, 1600),
                                      (20, 768, 50257), (512, 768, 2304), (1024, 768, 2304),
                                      (512, 768, 3072), (16, 1024, 3072), (32, 1600, 6400),
                                      (16, 4096, 1024), (16, 1600, 4800),
                                      (100, 48, 100), (333, 112, 260), (200, 32, 64), (64, 16, 52),
                                      (1024, 3072, 768), (1024, 1600, 4800),
                                      (16, 100, 52), (24, 768, 768), (16, 768, 1000),
                                      (48, 768, 2304), (33, 1600, 1600), (64, 3072, 768),
                                      (1024, 1024, 4096), (1024, 4096, 1024), (1100, 1600, 1600)])
def test_dense_many_rows_uses_mfma_gemm(rows, k, n):
    # rows >= 16 and K % 16 == 0 take the MFMA GEMM; tails in M and N are exercised.
    # (64, 6400, 1600), (16, 1024, 3072) and (32, 1600, 6400) cut the whole K range into
    # parts; (512, 768, 2304), (1024, 768, 2304) and (512, 768, 3072) have 288 / 576 / 384
    # tiles of 64x64 on 256 CUs and cut only the tiles of the last partial round.
    # K = 48 and 112 are not multiples of 32 and take k-tiles of 16 columns; K = 16 and 32 are a
    # single k-tile (the pipelined loop's shortest cases); (1024, 3072, 768) has a deep K on 192
    # tiles and is cut in four.  From 1024 rows on, products with enough 128x128 tiles run on the
    # bf16 matrix cores with input and weights cut into three bf16 parts each and all nine
    # products formed (exact): whole tiles for (1024, 1600, 4800) and (1024, 1024, 4096), tiles
    # cut in four along K for (1024, 4096, 1024) and (1100, 1600, 1600), whose last tile row is
    # ragged.
    # Up to 32 rows take the MFMA kernel of the decode batch: 16 rows its 16x16x4 form, with 16
    # rows of W per block where 32 would leave CUs idle ((16, 768, 2304), (16, 1024, 3072),
    # (16, 768, 1000) with a ragged last block) and 32 otherwise ((16, 1600, 4800); (16, 4096,
    # 1024) with K cut over blocks); 17..32 rows the 32x32x2 form ((32, 1600, 6400), (20, 768,
    # 50257), (24, 768, 768)); 33..64 rows that form with two tiles of input rows ((48, 768,
    # 2304), (33, 1600, 1600) and (64, 3072, 768) with K cut over blocks, (37, 64, 50) ragged,
    # (64, 16, 52) with a single step for eight wavefronts).  (16, 100, 52): K is no multiple
    # of 16, the row-streaming kernel.
    rng = np.random.default_rng(rows * 7 + n)
    x = rng.standard_normal(rows * k).astype(np.float32)
    w = (rng.standard_normal(n * k) * 0.02).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    got = hip_dense(x, rows, k, n, w, b)
    want = oracle.transposed_dense(x, rows, k, n, w, b)
    np.testing.assert_allclose(got, want, atol=3e-5, rtol=1e-5)


@pytest.mark.parametrize("rows,k,n", [(1024, 1024, 4096), (1024, 1600, 1600), (96, 768, 768)])
def test_dense_with_selection_weights_returns_the_inputs_bit_for_bit(rows, k, n):
    """W[o, :] is a unit vector, so out[r, o] must be exactly x[r, o % k] whatever the
    summation order: every other product is 0.  For the first two shapes the product runs on
    the bf16 matrix cores with x and W cut into three bf16 parts each (whole tiles; tiles cut
    in four along K): the parts of a value must add up to the value in all its 24 bits, at any
    exponent.  (96 rows: the f32 matrix cores, for comparison.)"""
    rng = np.random.default_rng(rows + n)
    x = (rng.standard_normal(rows * k) * 10.0 ** rng.uniform(-6, 6, rows * k)).astype(np.float32)
    x[::97] = np.float32(1.0) + np.float32(2.0) ** -23  # all-but-one low bits clear
    x[1::97] = np.nextafter(np.float32(2.0), np.float32(0.0))  # 24 ones
    w = np.zeros((n, k), np.float32)
    w[np.arange(n), np.arange(n) % k] = 1.0
    got = hip_dense(x, rows, k, n, w.reshape(-1), np.zeros(n, np.float32)).reshape(rows, n)
    want = x.reshape(rows, k)[:, np.arange(n) % k]
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("rows,k,n", [(1024, 1024, 4096), (1024, 4096, 1024), (48, 768, 2304)])
def test_dense_keeps_infinities_and_nans_of_the_input(rows, k, n):
    """dot (cpu.rs:231-254) carries an infinite or NaN input or weight into the sums as f32
    arithmetic does: +inf times a positive weight is +inf, opposite infinities in one row give
    NaN, inf times a zero weight gives NaN, a NaN stays a NaN, and rows without such a value are
    untouched.  48 rows run on the f32 matrix cores.  The first two shapes run on the bf16 matrix
    cores with x AND W cut into three bf16 parts each (whole tiles; tiles cut in four along K),
    where a zero part times an infinity would be NaN: a tile that has met an infinity is computed
    again in f32 arithmetic, so the result is the reference's there as well."""
    rng = np.random.default_rng(rows + k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    x[3, 5] = np.inf           # one infinity: the sign of w[o, 5] decides
    x[7, 11] = -np.inf
    x[9, 2], x[9, k - 1] = np.inf, -np.inf   # both in a row: inf - inf somewhere, or +-inf
    x[12, 40] = np.nan
    x[rows - 1, k - 3] = np.inf
    w[5, 5] = 0.0              # inf * 0 is NaN in f32 as well
    w[n - 2, 17] = -np.inf     # an infinite weight: every row's output n - 2, by the sign of x[:, 17]
    got = hip_dense(x.reshape(-1), rows, k, n, w.reshape(-1), b).reshape(rows, n)
    with np.errstate(invalid="ignore"):
        want = oracle.transposed_dense(x.reshape(-1), rows, k, n, w.reshape(-1), b).reshape(rows, n)
    assert np.isnan(want[3, 5]) and np.isinf(want[3]).sum() >= n - 2 and np.isnan(want[12]).all()
    assert np.isinf(want[:, n - 2]).sum() >= rows - 6
    fin = np.isfinite(want)
    np.testing.assert_array_equal(np.isfinite(got), fin)
    np.testing.assert_allclose(got[fin], want[fin], atol=3e-5, rtol=1e-5)
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(np.isposinf(got), np.isposinf(want))
    np.testing.assert_array_equal(np.isneginf(got), np.isneginf(want))


def test_dense_reference_unit_vector():
    # src/models/cpu.rs:312-327
    x, weight = patterned(6, 0.2), patterned(12, 0.1)
    bias = np.array([0.5, -0.25, 0.125, 0.0], np.float32)
    t = oracle.transpose_in_out(weight, 3, 4)
    np.testing.assert_allclose(hip_dense(x, 2, 3, 4, t, bias), oracle.dense(x, 2, 3, 4, weight, bias),
                               atol=1e-6, rtol=0)


@pytest.mark.parametrize("rows,cols", [(1, 4), (1, 768), (3, 1600), (5, 37), (2, 6400)])
def test_layer_norm_matches_oracle(rows, cols):
    rng = np.random.default_rng(cols)
    x = (rng.standard_normal(rows * cols) * 3 + 1.5).astype(np.float32)
    g = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    got = x.copy()
    ok(L().pg_op_layer_norm(0, _lib.f32p(got), rows, cols, _lib.f32p(g), _lib.f32p(b), 1e-5))
    np.testing.assert_allclose(got, oracle.layer_norm(x, rows, cols, g, b, 1e-5), atol=5e-6, rtol=1e-5)


def test_gelu_softmax_add_match_oracle():
    x = np.linspace(-8, 8, 4001).astype(np.float32)
    got = x.copy()
    ok(L().pg_op_gelu(0, _lib.f32p(got), got.size))
    np.testing.assert_allclose(got, oracle.gelu(x), atol=1e-6, rtol=1e-5)
    rng = np.random.default_rng(5)
    for n in [1, 2, 33, 1024, 5000]:
        v = (rng.standard_normal(n) * 4).astype(np.float32)
        got = v.copy()
        ok(L().pg_op_softmax(0, _lib.f32p(got), 1, n))
        np.testing.assert_allclose(got, oracle.softmax(v), atol=1e-7, rtol=1e-5)
    a, b = patterned(1000, 0.5), patterned(1000, -0.25)
    got = a.copy()
    ok(L().pg_op_add(0, _lib.f32p(got), _lib.f32p(b), got.size))
    np.testing.assert_array_equal(got, oracle.add(a, b))


def oracle_attention(qkv, pos, keys, values, P, H, hd):
    """cached_self_attention_into restated with the oracle's softmax (rust.rs:1662-1741)."""
    C_ = H * hd
    k, v = keys.reshape(H, P, hd).copy(), values.reshape(H, P, hd).copy()
    k[:, pos] = qkv[C_:2 * C_].reshape(H, hd)
    v[:, pos] = qkv[2 * C_:].reshape(H, hd)
    out = np.zeros(C_, np.float32)
    scale = np.float32(1.0) / np.sqrt(np.float32(hd))
    for h in range(H):
        s = np.array([oracle.dot_scalar(qkv[h * hd:(h + 1) * hd], k[h, j]) for j in range(pos + 1)],
                     np.float32) * scale
        p = oracle.softmax(s)
        out[h * hd:(h + 1) * hd] = (p[:, None].astype(np.float64) * v[h, :pos + 1]).sum(0)
    return out, k, v


@pytest.mark.parametrize("H,hd,P,pos", [(2, 2, 5, 0), (2, 2, 5, 4), (12, 64, 1024, 0), (12, 64, 1024, 31),
                                        (25, 64, 1024, 1023), (16, 64, 1024, 383), (3, 12, 64, 40),
                                        (1, 64, 128, 17)])
def test_attention_decode_matches_oracle(H, hd, P, pos):
    rng = np.random.default_rng(H * 1000 + pos)
    C_ = H * hd
    qkv = rng.standard_normal(3 * C_).astype(np.float32)
    keys = rng.standard_normal(H * P * hd).astype(np.float32)
    values = rng.standard_normal(H * P * hd).astype(np.float32)
    want, wk, wv = oracle_attention(qkv, pos, keys, values, P, H, hd)
    out = np.empty(C_, np.float32)
    k, v = keys.copy(), values.copy()
    ok(L().pg_op_attention_decode(0, _lib.f32p(qkv), pos, _lib.f32p(k), _lib.f32p(v), P, H, hd,
                                  _lib.f32p(out)))
    np.testing.assert_allclose(out, want, atol=2e-5, rtol=1e-4)
    np.testing.assert_array_equal(k.reshape(H, P, hd), wk)   # K/V append at kv_index
    np.testing.assert_array_equal(v.reshape(H, P, hd), wv)


def test_argmax_rules_match_oracle():
    inf, nan = float("inf"), float("nan")
    cases = [[1.0, 3.0, 3.0, 2.0], [-inf, -inf], [nan, nan, nan], [1.0, nan, 0.5],
             [nan, 1.0, inf, inf], [-5.0]]
    rng = np.random.default_rng(9)
    big = rng.standard_normal(50257).astype(np.float32)
    big[[777, 40000]] = big.max() + 1.0  # a tie far apart: lowest index wins
    cases.append(big)
    cases.append(np.full(50257, -inf, np.float32))
    for c in cases:
        v = np.asarray(c, np.float32)
        out = C.c_uint32()
        ok(L().pg_op_argmax(0, _lib.f32p(v), v.size, C.byref(out)))
        assert out.value == oracle.argmax_logits(v)
