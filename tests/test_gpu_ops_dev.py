"""The op-level seam on device operands (what a second model family would call between its own
steps): each op against the oracle's restatement of src/models/cpu.rs, the [in,out] dense
projection (cpu.rs:77-97) and the multi-query attention of the reference's Whisper model
(src/models/whisper/model.rs:1262-1357), chained without leaving the device."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import DeviceArray
from puppygrad_amd import _lib

pytestmark = pytest.mark.gpu


def ok(status):
    assert status == 0, _lib.load().pg_last_error_message().decode()


def attention_values(q, k, v, heads, causal):
    """attention_values_into restated in float64 with the oracle's softmax per row."""
    Tq, state = q.shape
    Tk = k.shape[0]
    hd = state // heads
    out = np.zeros((Tq, state), np.float64)
    for h in range(heads):
        sl = slice(h * hd, (h + 1) * hd)
        for i in range(Tq):
            n = min(i + 1, Tk) if causal else Tk
            s = (k[:n, sl].astype(np.float64) @ q[i, sl].astype(np.float64)) / np.sqrt(np.float32(hd))
            p = oracle.softmax(s.astype(np.float32)).astype(np.float64)
            out[i, sl] = p @ v[:n, sl].astype(np.float64)
    return out


@pytest.mark.parametrize("rows,in_f,out_f", [(1, 8, 5), (3, 100, 257), (7, 384, 1536), (20, 768, 768),
                                             (1, 4096, 33), (5, 1, 300)])
def test_dense_with_in_out_weights_matches_oracle(rows, in_f, out_f):
    rng = np.random.default_rng(rows * 1000 + in_f)
    x = rng.standard_normal((rows, in_f)).astype(np.float32)
    w = (rng.standard_normal((in_f, out_f)) / np.sqrt(in_f)).astype(np.float32)
    b = rng.standard_normal(out_f).astype(np.float32)
    dx, dw, db, dy = DeviceArray(x), DeviceArray(w), DeviceArray(b), DeviceArray(np.zeros((rows, out_f)))
    ok(_lib.load().pg_op_dense_in_out_dev(0, None, dx.ptr, rows, in_f, out_f, dw.ptr, db.ptr, dy.ptr))
    want = oracle.dense(x, rows, in_f, out_f, w, b).reshape(rows, out_f)
    np.testing.assert_allclose(dy.download(), want, atol=2e-5, rtol=1e-4)
    # the same product through the [out,in] entry point on the transposed weights
    dwt = DeviceArray(np.ascontiguousarray(w.T))
    ok(_lib.load().pg_op_dense_dev(0, None, dx.ptr, rows, in_f, out_f, dwt.ptr, db.ptr, dy.ptr))
    np.testing.assert_allclose(dy.download(), want, atol=2e-5, rtol=1e-4)
    for d in (dx, dw, db, dy, dwt):
        d.free()


@pytest.mark.parametrize("rows", [2, 5, 8, 16, 17, 31, 33, 47, 64, 65])
def test_dense_on_device_over_the_small_batch_forms(rows):
    """2..64 rows take the small-batch projection kernel in its 16-row, 32-row and two-tile forms
    (65: the tile GEMM), with ragged row blocks (N no multiple of the block height), a single
    k step for eight wavefronts (K = 16) and N below one block."""
    lib = _lib.load()
    for in_f, out_f in [(768, 2304), (1600, 100), (16, 52), (160, 1000), (64, 7)]:
        rng = np.random.default_rng(rows * 131 + in_f + out_f)
        x = rng.standard_normal((rows, in_f)).astype(np.float32)
        w = (rng.standard_normal((out_f, in_f)) / np.sqrt(in_f)).astype(np.float32)
        b = rng.standard_normal(out_f).astype(np.float32)
        dx, dw, db, dy = DeviceArray(x), DeviceArray(w), DeviceArray(b), DeviceArray(np.zeros((rows, out_f)))
        ok(lib.pg_op_dense_dev(0, None, dx.ptr, rows, in_f, out_f, dw.ptr, db.ptr, dy.ptr))
        want = x.astype(np.float64) @ w.astype(np.float64).T + b
        np.testing.assert_allclose(dy.download(), want, atol=3e-5, rtol=1e-5, err_msg=f"{rows}x{in_f}x{out_f}")
        for d in (dx, dw, db, dy):
            d.free()


@pytest.mark.parametrize("rows,in_f,out_f", [(1, 384, 51865), (2, 100, 37), (1, 16, 8), (3, 1280, 1000),
                                             (1, 7, 5), (12, 384, 1536), (40, 768, 2304), (150, 1280, 5120),
                                             (300, 1024, 8200)])
def test_quantized_rows_and_quantized_dense_match_oracle(rows, in_f, out_f):
    """QuantizedRows::from_f32 bit for bit (incl. an all-zero row and a row whose largest value is
    negative), then the quantised projection against quantized_dot (cpu.rs:99-117, 173-184), with
    a bias and without one (the Whisper logits, model.rs:1528).  Several rows with a row length
    that is a multiple of 64 take the matrix-core kernels: 3 and 12 rows the 32-row kernel's two
    forms, 40 rows the f32-core tiles, 150 and 300 rows the bf16-core tiles (whole 128 x 128
    tiles; a ragged last tile row and column)."""
    rng = np.random.default_rng(in_f * 7 + out_f)
    w = (rng.standard_normal((out_f, in_f)) / np.sqrt(in_f)).astype(np.float32)
    w[0] = 0.0
    w[out_f - 1, 0] = -3.0
    x = rng.standard_normal((rows, in_f)).astype(np.float32)
    b = rng.standard_normal(out_f).astype(np.float32)
    lib = _lib.load()
    dw, dq, ds = DeviceArray(w), DeviceArray(np.zeros((out_f, in_f)), np.int8), DeviceArray(np.zeros(out_f))
    ok(lib.pg_op_quantize_rows_dev(0, None, dw.ptr, out_f, in_f, dq.ptr, ds.ptr))
    q_want, s_want = oracle.quantize_rows(w, out_f, in_f)
    np.testing.assert_array_equal(dq.download(), q_want)
    np.testing.assert_array_equal(ds.download(), s_want)
    dx, db, dy = DeviceArray(x), DeviceArray(b), DeviceArray(np.zeros((rows, out_f)))
    idx = np.unique(np.concatenate([np.arange(min(out_f, 40)), rng.integers(0, out_f, 60), [out_f - 1]]))
    dots = np.array([[oracle.quantized_dot(x[r], q_want, s_want, int(o)) for o in idx] for r in range(rows)],
                    np.float32)
    ok(lib.pg_op_quantized_dense_dev(0, None, dx.ptr, rows, in_f, out_f, dq.ptr, ds.ptr, db.ptr, dy.ptr))
    np.testing.assert_allclose(dy.download()[:, idx], dots + b[idx], atol=2e-5, rtol=1e-4)
    ok(lib.pg_op_quantized_dense_dev(0, None, dx.ptr, rows, in_f, out_f, dq.ptr, ds.ptr, None, dy.ptr))
    np.testing.assert_allclose(dy.download()[:, idx], dots, atol=2e-5, rtol=1e-4)
    assert lib.pg_op_quantized_dense_dev(0, None, dx.ptr, rows, 0, out_f, dq.ptr, ds.ptr, None, dy.ptr) == _lib.PG_INVALID_INPUT
    assert lib.pg_op_quantize_rows_dev(0, None, dw.ptr, out_f, in_f, None, ds.ptr) == _lib.PG_INVALID_INPUT
    for d in (dw, dq, ds, dx, db, dy):
        d.free()


@pytest.mark.parametrize("rows,in_f,out_f", [(12, 384, 1536), (150, 1280, 5120)])
def test_quantized_dense_keeps_infinities_and_nans_of_the_input(rows, in_f, out_f):
    """quantized_dot (cpu.rs:173-184) in f32 arithmetic: an infinite input gives +-inf by the sign
    of the weight (NaN against a zero weight), a NaN gives NaN.  12 rows run on the 32-row kernel
    and 150 on the tile kernel, both on the bf16 matrix cores with the inputs cut into three bf16
    parts: a non-finite value has to stay whole in the first part."""
    rng = np.random.default_rng(rows)
    w = (rng.standard_normal((out_f, in_f)) / np.sqrt(in_f)).astype(np.float32)
    x = rng.standard_normal((rows, in_f)).astype(np.float32)
    x[1, 3] = np.inf
    x[2, 7] = -np.inf
    x[4, 9] = np.nan
    x[rows - 1, in_f - 1] = np.inf
    lib = _lib.load()
    dw, dq, ds = DeviceArray(w), DeviceArray(np.zeros((out_f, in_f)), np.int8), DeviceArray(np.zeros(out_f))
    ok(lib.pg_op_quantize_rows_dev(0, None, dw.ptr, out_f, in_f, dq.ptr, ds.ptr))
    q, sc = dq.download(), ds.download()
    dx, dy = DeviceArray(x), DeviceArray(np.zeros((rows, out_f)))
    ok(lib.pg_op_quantized_dense_dev(0, None, dx.ptr, rows, in_f, out_f, dq.ptr, ds.ptr, None, dy.ptr))
    got = dy.download()
    with np.errstate(invalid="ignore"):
        want = x @ (q.astype(np.float32) * sc[:, None]).T
    assert np.isinf(want[1]).sum() > out_f // 2 and np.isnan(want[4]).all()
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(np.isposinf(got), np.isposinf(want))
    np.testing.assert_array_equal(np.isneginf(got), np.isneginf(want))
    fin = np.isfinite(want)
    np.testing.assert_allclose(got[fin], want[fin], atol=5e-5, rtol=1e-4)
    for d in (dw, dq, ds, dx, dy):
        d.free()


@pytest.mark.parametrize("Tq,Tk,state,heads,causal", [(1, 1, 8, 2, 0), (5, 5, 24, 3, 1), (6, 1500, 384, 6, 0),
                                                      (40, 40, 384, 6, 1), (3, 700, 1280, 20, 0),
                                                      (9, 4, 64, 1, 1), (2, 33, 512, 2, 0)])
def test_attention_rows_matches_the_reference_formula(Tq, Tk, state, heads, causal):
    rng = np.random.default_rng(Tq * 100 + Tk)
    q = rng.standard_normal((Tq, state)).astype(np.float32)
    k = rng.standard_normal((Tk, state)).astype(np.float32)
    v = rng.standard_normal((Tk, state)).astype(np.float32)
    dq, dk, dv, dout = DeviceArray(q), DeviceArray(k), DeviceArray(v), DeviceArray(np.zeros((Tq, state)))
    ok(_lib.load().pg_op_attention_dev(0, None, dq.ptr, dk.ptr, dv.ptr, Tq, Tk, state, heads, causal, dout.ptr))
    np.testing.assert_allclose(dout.download(), attention_values(q, k, v, heads, bool(causal)),
                               atol=2e-5, rtol=1e-4)
    for d in (dq, dk, dv, dout):
        d.free()


def test_an_encoder_style_block_stays_on_the_device():
    """LayerNorm -> q/k/v projections -> attention over all keys -> projection + residual ->
    LayerNorm -> fc + GELU -> projection + residual -> argmax, op by op on device buffers,
    against the same chain of oracle ops on the host."""
    rng = np.random.default_rng(7)
    T, S, H, I = 12, 128, 4, 512
    lib = _lib.load()
    x = rng.standard_normal((T, S)).astype(np.float32)
    p = {n: (rng.standard_normal(shape) * 0.1).astype(np.float32) for n, shape in
         [("wq", (S, S)), ("wk", (S, S)), ("wv", (S, S)), ("wo", (S, S)), ("w1", (I, S)), ("w2", (S, I)),
          ("bq", S), ("bk", S), ("bv", S), ("bo", S), ("b1", I), ("b2", S), ("g1", S), ("be1", S),
          ("g2", S), ("be2", S)]}
    # host chain with the oracle's ops
    xn = oracle.layer_norm(x, T, S, p["g1"], p["be1"], 1e-5).reshape(T, S)
    q = oracle.transposed_dense(xn, T, S, S, p["wq"], p["bq"]).reshape(T, S)
    k = oracle.transposed_dense(xn, T, S, S, p["wk"], p["bk"]).reshape(T, S)
    v = oracle.transposed_dense(xn, T, S, S, p["wv"], p["bv"]).reshape(T, S)
    att = attention_values(q, k, v, H, False).astype(np.float32)
    x1 = oracle.add(x.reshape(-1), oracle.transposed_dense(att, T, S, S, p["wo"], p["bo"])).reshape(T, S)
    xn2 = oracle.layer_norm(x1, T, S, p["g2"], p["be2"], 1e-5).reshape(T, S)
    h = oracle.gelu(oracle.transposed_dense(xn2, T, S, I, p["w1"], p["b1"]))
    want = oracle.add(x1.reshape(-1), oracle.transposed_dense(h.reshape(T, I), T, I, S, p["w2"], p["b2"]))
    # device chain
    d = {n: DeviceArray(a) for n, a in p.items()}
    dx, dxn = DeviceArray(x), DeviceArray(x)
    dq, dk, dv, datt, dtmp = (DeviceArray(np.zeros((T, S))) for _ in range(5))
    dh = DeviceArray(np.zeros((T, I)))
    did = DeviceArray(np.zeros(1, np.uint32), dtype=np.uint32)
    ok(lib.pg_op_layer_norm_dev(0, None, dxn.ptr, T, S, d["g1"].ptr, d["be1"].ptr, 1e-5))
    for w, b, dst in (("wq", "bq", dq), ("wk", "bk", dk), ("wv", "bv", dv)):
        ok(lib.pg_op_dense_dev(0, None, dxn.ptr, T, S, S, d[w].ptr, d[b].ptr, dst.ptr))
    ok(lib.pg_op_attention_dev(0, None, dq.ptr, dk.ptr, dv.ptr, T, T, S, H, 0, datt.ptr))
    ok(lib.pg_op_dense_dev(0, None, datt.ptr, T, S, S, d["wo"].ptr, d["bo"].ptr, dtmp.ptr))
    ok(lib.pg_op_add_dev(0, None, dx.ptr, dtmp.ptr, T * S))
    ok(lib.pg_device_upload(0, dxn.ptr, dx.download().ctypes.data_as(C.c_void_p), T * S * 4))
    ok(lib.pg_op_layer_norm_dev(0, None, dxn.ptr, T, S, d["g2"].ptr, d["be2"].ptr, 1e-5))
    ok(lib.pg_op_dense_dev(0, None, dxn.ptr, T, S, I, d["w1"].ptr, d["b1"].ptr, dh.ptr))
    ok(lib.pg_op_gelu_dev(0, None, dh.ptr, T * I))
    ok(lib.pg_op_dense_dev(0, None, dh.ptr, T, I, S, d["w2"].ptr, d["b2"].ptr, dtmp.ptr))
    ok(lib.pg_op_add_dev(0, None, dx.ptr, dtmp.ptr, T * S))
    got = dx.download().reshape(-1)
    np.testing.assert_allclose(got, want, atol=1e-4, rtol=1e-3)
    ok(lib.pg_op_softmax_dev(0, None, dx.ptr, T, S))
    np.testing.assert_allclose(dx.download(), np.stack([oracle.softmax(r) for r in got.reshape(T, S)]),
                               atol=1e-6, rtol=1e-4)
    ok(lib.pg_op_argmax_dev(0, None, dx.ptr, T * S, did.ptr))
    assert int(did.download()[0]) == oracle.argmax_logits(dx.download().reshape(-1))


def test_device_ops_refuse_bad_shapes():
    lib = _lib.load()
    one = DeviceArray(np.zeros(8))
    assert lib.pg_op_dense_in_out_dev(0, None, one.ptr, 1, 5000, 4, one.ptr, one.ptr, one.ptr) == _lib.PG_INVALID_INPUT
    assert lib.pg_op_attention_dev(0, None, one.ptr, one.ptr, one.ptr, 1, 1, 10, 3, 0, one.ptr) == _lib.PG_INVALID_INPUT
    assert b"state must be heads * head_dim" in lib.pg_last_error_message()
    assert lib.pg_op_attention_dev(0, None, one.ptr, one.ptr, one.ptr, 1, 0, 8, 2, 0, one.ptr) == _lib.PG_INVALID_INPUT
    assert lib.pg_op_layer_norm_dev(0, None, None, 1, 8, one.ptr, one.ptr, 1e-5) == _lib.PG_INVALID_INPUT
    # the limits a row staged in LDS sets, refused before any launch
    assert lib.pg_op_layer_norm_dev(0, None, one.ptr, 1, 16321, one.ptr, one.ptr, 1e-5) == _lib.PG_INVALID_INPUT
    assert b"cols must be in [1,16320]" in lib.pg_last_error_message()
    assert lib.pg_op_dense_dev(0, None, one.ptr, 1, 16321, 4, one.ptr, one.ptr, one.ptr) == _lib.PG_INVALID_INPUT
    assert b"in_features must be in [1,16320]" in lib.pg_last_error_message()
    assert lib.pg_op_dense_dev(0, None, one.ptr, (1 << 20) + 1, 8, 4, one.ptr, one.ptr, one.ptr) == _lib.PG_INVALID_INPUT
    assert lib.pg_op_attention_decode_noalloc(0, None, one.ptr, 0, one.ptr, one.ptr, 16321, 2, 4, one.ptr) == _lib.PG_INVALID_INPUT
    assert b"max_seq_len in [1,16320]" in lib.pg_last_error_message()
    # dense without a bias: only the quantised projection takes NULL
    assert lib.pg_op_dense_dev(0, None, one.ptr, 1, 8, 1, one.ptr, None, one.ptr) == _lib.PG_INVALID_INPUT
    one.free()


def test_dense_in_out_more_rows_than_one_launch_holds():
    """[in,out] dense with 262,200 rows of 2 values: the rows go out in two launches (a launch's
    second grid dimension ends at 65535 blocks of four rows)."""
    rows, in_f, out_f = 262200, 2, 3
    rng = np.random.default_rng(9)
    x = rng.standard_normal((rows, in_f)).astype(np.float32)
    w = rng.standard_normal((in_f, out_f)).astype(np.float32)
    b = rng.standard_normal(out_f).astype(np.float32)
    dx, dw, db, dy = DeviceArray(x), DeviceArray(w), DeviceArray(b), DeviceArray(np.zeros((rows, out_f)))
    ok(_lib.load().pg_op_dense_in_out_dev(0, None, dx.ptr, rows, in_f, out_f, dw.ptr, db.ptr, dy.ptr))
    np.testing.assert_allclose(dy.download(), x @ w + b, atol=1e-5, rtol=1e-5)
    for d in (dx, dw, db, dy):
        d.free()
