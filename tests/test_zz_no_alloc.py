"""The entry point that allocates nothing: pg_op_attention_decode_noalloc against
pg_op_attention_decode (cached_self_attention_into, src/models/gpt2/rust.rs:1662-1741) on the
same inputs, operands in device buffers, two calls in a row with the second one smaller (the
fixed scratch array still holds the first call's partial results)."""
import ctypes as C

import numpy as np
import pytest

from helpers import DeviceArray
from puppygrad_amd import _lib

pytestmark = pytest.mark.gpu


def attention_case(seed, H, hd, P, pos):
    rng = np.random.default_rng(seed)
    C_ = H * hd
    qkv = rng.standard_normal(3 * C_).astype(np.float32)
    keys = np.zeros((H, P, hd), np.float32)
    values = np.zeros((H, P, hd), np.float32)
    keys[:, :pos] = rng.standard_normal((H, pos, hd))
    values[:, :pos] = rng.standard_normal((H, pos, hd))
    return qkv, keys, values


def run_existing(qkv, keys, values, pos, H, hd, P):
    lib = _lib.load()
    k, v = keys.copy(), values.copy()
    out = np.empty(H * hd, np.float32)
    st = lib.pg_op_attention_decode(0, _lib.f32p(qkv), pos, _lib.f32p(k), _lib.f32p(v), P, H, hd,
                                    _lib.f32p(out))
    assert st == 0, lib.pg_last_error_message()
    return out, k, v


def run_noalloc(qkv, keys, values, pos, H, hd, P):
    lib = _lib.load()
    dq, dk, dv = DeviceArray(qkv), DeviceArray(keys), DeviceArray(values)
    dout = DeviceArray(np.zeros(H * hd, np.float32))
    st = lib.pg_op_attention_decode_noalloc(0, None, dq.ptr, pos, dk.ptr, dv.ptr, P, H, hd, dout.ptr)
    assert st == 0, lib.pg_last_error_message()
    got = dout.download(), dk.download(), dv.download()
    for d in (dq, dk, dv, dout):
        d.free()
    return got


def test_attention_decode_without_allocation_matches_the_allocating_entry_point():
    # two calls in a row; the second is smaller in every dimension the scratch depends on
    for seed, H, hd, P, pos in [(1, 25, 64, 1024, 900), (2, 12, 64, 256, 37), (3, 3, 20, 96, 50),
                                (4, 16, 64, 1024, 1023), (5, 2, 64, 64, 0)]:
        qkv, keys, values = attention_case(seed, H, hd, P, pos)
        want = run_existing(qkv, keys, values, pos, H, hd, P)
        got = run_noalloc(qkv, keys, values, pos, H, hd, P)
        for g, w, what in zip(got, want, ("out", "keys", "values")):
            np.testing.assert_array_equal(g, w, err_msg=f"{what} seed {seed}")  # same kernels: same bits
        # and equal to cached_self_attention_into (rust.rs:1662-1741) in float64
        C_ = H * hd
        k, v = keys.astype(np.float64), values.astype(np.float64)
        q = qkv[:C_].astype(np.float64).reshape(H, hd)
        k[:, pos] = qkv[C_:2 * C_].reshape(H, hd)
        v[:, pos] = qkv[2 * C_:].reshape(H, hd)
        s = np.einsum("hd,hkd->hk", q, k[:, :pos + 1]) / np.sqrt(hd)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        ref_out = np.einsum("hk,hkd->hd", p, v[:, :pos + 1]).reshape(-1)
        np.testing.assert_allclose(got[0], ref_out, atol=1e-4, rtol=1e-3)


def test_attention_decode_without_allocation_refuses_what_its_scratch_cannot_hold():
    lib = _lib.load()
    one = DeviceArray(np.zeros(4, np.float32))
    # 5000 = 50 heads x 100 > 4096 columns; 300 heads > 256: refused before any pointer is used
    for H, hd in ((50, 100), (300, 8)):
        st = lib.pg_op_attention_decode_noalloc(0, None, one.ptr, 0, one.ptr, one.ptr, 8, H, hd, one.ptr)
        assert st == _lib.PG_INVALID_INPUT
        assert b"exceeds the fixed scratch" in lib.pg_last_error_message()
    st = lib.pg_op_attention_decode_noalloc(0, None, one.ptr, 8, one.ptr, one.ptr, 8, 2, 64, one.ptr)
    assert st == _lib.PG_INVALID_INPUT and b"cache is full at seq_len 8" in lib.pg_last_error_message()
    one.free()
