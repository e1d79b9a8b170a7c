"""Pins the oracle's cpu.rs restatement: the reference's own unit-test vectors
(src/models/cpu.rs:303-345, src/runtime/thread_pool.rs:230-256), float64 closed
forms, and torch's CPU library routines."""
import numpy as np
import torch
import torch.nn.functional as F

import oracle
from puppygrad_amd.synth import patterned


def test_dot_matches_scalar_reference():
    # cpu.rs:304-309: len 37 exercises the 8-lane body and the scalar tail
    a, b = patterned(37, 0.013), patterned(37, -0.021)
    assert abs(oracle.dot(a, b) - oracle.dot_scalar(a, b)) <= 1e-6
    exact = float(np.dot(a.astype(np.float64), b.astype(np.float64)))
    assert abs(oracle.dot(a, b) - exact) <= 1e-6
    # the pattern's integers are i*17+11 mod 23 - 11 (rust.rs appendix values)
    assert [round(float(v) / 0.013) for v in a[:12]] == [0, -6, 11, 5, -1, -7, 10, 4, -2, -8, 9, 3]


def test_dot_lengths_and_tail():
    rng = np.random.default_rng(1)
    for n in [0, 1, 7, 8, 9, 15, 16, 17, 64, 768, 1600, 6400]:
        a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
        exact = float(np.dot(a.astype(np.float64), b.astype(np.float64)))
        scale = float(np.abs(a.astype(np.float64) * b).sum()) + 1e-30
        assert abs(oracle.dot(a, b) - exact) <= 2e-6 * scale
        assert abs(oracle.dot_scalar(a, b) - exact) <= 2e-6 * scale


def test_transposed_dense_matches_dense():
    # cpu.rs:312-327
    x, weight = patterned(6, 0.2), patterned(12, 0.1)
    bias = np.array([0.5, -0.25, 0.125, 0.0], np.float32)
    transposed = oracle.transpose_in_out(weight, 3, 4)
    d = oracle.dense(x, 2, 3, 4, weight, bias)
    t = oracle.transposed_dense(x, 2, 3, 4, transposed, bias)
    np.testing.assert_allclose(d, t, atol=1e-6, rtol=0)
    exact = x.astype(np.float64).reshape(2, 3) @ weight.astype(np.float64).reshape(3, 4) + bias
    np.testing.assert_allclose(t.reshape(2, 4), exact, atol=1e-6, rtol=0)
    # transpose is the [in,out] -> [out,in] permutation
    np.testing.assert_array_equal(transposed.reshape(4, 3), weight.reshape(3, 4).T)


def test_dense_against_torch_linear():
    rng = np.random.default_rng(2)
    for rows, k, n in [(1, 768, 96), (3, 100, 7), (2, 1600, 33)]:
        x = rng.standard_normal((rows, k)).astype(np.float32)
        w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32)
        got = oracle.transposed_dense(x, rows, k, n, w, b).reshape(rows, n)
        want = F.linear(torch.from_numpy(x).double(), torch.from_numpy(w).double(),
                        torch.from_numpy(b).double()).numpy()
        np.testing.assert_allclose(got, want, atol=2e-6, rtol=1e-5)


def test_layer_norm_against_torch_and_closed_form():
    rng = np.random.default_rng(3)
    for rows, cols in [(1, 4), (3, 768), (2, 1600), (5, 37)]:
        x = (rng.standard_normal((rows, cols)) * 3 + 1.5).astype(np.float32)
        g = rng.standard_normal(cols).astype(np.float32)
        b = rng.standard_normal(cols).astype(np.float32)
        got = oracle.layer_norm(x, rows, cols, g, b, 1e-5).reshape(rows, cols)
        want = F.layer_norm(torch.from_numpy(x).double(), (cols,), torch.from_numpy(g).double(),
                            torch.from_numpy(b).double(), 1e-5).numpy()
        np.testing.assert_allclose(got, want, atol=5e-6, rtol=1e-5)
    # closed form: a constant row has zero variance, so y = beta; eps sits inside the sqrt
    x = np.full((1, 8), 2.5, np.float32)
    out = oracle.layer_norm(x, 1, 8, np.ones(8, np.float32), np.full(8, 0.25, np.float32), 1e-5)
    np.testing.assert_allclose(out.reshape(-1), 0.25, atol=1e-7)
    x = np.array([[1.0, -1.0]], np.float32)  # mean 0, biased var 1 -> 1/sqrt(1+eps)
    out = oracle.layer_norm(x, 1, 2, np.ones(2, np.float32), np.zeros(2, np.float32), 0.21)
    np.testing.assert_allclose(out.reshape(-1), np.array([1, -1]) / np.sqrt(1.21), atol=1e-7)


def test_gelu_against_torch_tanh_form():
    x = np.linspace(-8, 8, 4001).astype(np.float32)
    got = oracle.gelu(x)
    want = F.gelu(torch.from_numpy(x).double(), approximate="tanh").numpy()
    np.testing.assert_allclose(got, want, atol=2e-6, rtol=1e-5)
    assert oracle.gelu(np.zeros(1, np.float32))[0] == 0.0


def test_softmax_against_torch():
    rng = np.random.default_rng(4)
    for n in [1, 2, 33, 1024]:
        x = (rng.standard_normal(n) * 4).astype(np.float32)
        got = oracle.softmax(x)
        want = torch.softmax(torch.from_numpy(x).double(), 0).numpy()
        np.testing.assert_allclose(got, want, atol=1e-7, rtol=1e-5)
        assert abs(float(got.sum()) - 1.0) < 1e-5
    # max-subtracted: huge inputs do not overflow
    got = oracle.softmax(np.array([1000.0, 1000.0], np.float32))
    np.testing.assert_allclose(got, [0.5, 0.5])


def test_add_in_place():
    a, b = patterned(10, 0.5), patterned(10, -0.25)
    np.testing.assert_array_equal(oracle.add(a, b), a + b)


def test_thread_pool_chunk_order():
    # thread_pool.rs:231-238: 10 items in chunks of 3 on 4 threads come back in order
    ids = oracle.pool_chunk_ids(4, 10, 3)
    np.testing.assert_array_equal(ids, np.arange(10) // 3)
    # thread_pool.rs:241-246: single thread, 7 items in chunks of 2 -> 4 chunks
    np.testing.assert_array_equal(oracle.pool_chunk_ids(1, 7, 2), [0, 0, 1, 1, 2, 2, 3])
    # more threads than chunks, chunk size 0 is clamped to 1 (thread_pool.rs:120)
    np.testing.assert_array_equal(oracle.pool_chunk_ids(8, 3, 0), [0, 1, 2])
    assert oracle.pool_chunk_ids(3, 0, 4).size == 0
