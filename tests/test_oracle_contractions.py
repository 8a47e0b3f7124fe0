"""Pins the oracle's dense GEMM and attention (checkers for the layer runner):
FP64 closed forms, the compiled reference at its own test tolerance
(tests/test_cpu_kernels.c:128-147 holds gemm_f16w to 1e-5; its summation order
is SIMD-dependent), and structural invariants of causal GQA attention."""
import ctypes as C

import numpy as np
import pytest

import oracle
from conftest import scaled_rel_err

needs_ref = pytest.mark.skipif(oracle.ref is None, reason="oracle/_ref not built here")
f32p = C.POINTER(C.c_float)


@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (3, 64, 1536), (7, 512, 3584), (13, 100, 131)])
def test_gemm_closed_form_and_reference(M, N, K):
    x = oracle.normal_f32((M, K), 1 + M)
    w = oracle.normal_f16((N, K), 2 + N, std=K ** -0.5)
    b = oracle.normal_f16((N,), 3, std=0.1)
    got = oracle.gemm_f16w(x, w, b)
    want = x.astype(np.float64) @ oracle.widen(w).astype(np.float64).T + oracle.widen(b)
    assert scaled_rel_err(got, want) <= 1e-6
    assert scaled_rel_err(oracle.gemm_f16w(x, w), want - oracle.widen(b)) <= 1e-6
    if oracle.ref is not None:
        r = np.empty((M, N), np.float32)
        assert oracle.ref.vv_gemm_f16w_cpu(x.ctypes.data_as(f32p), w.ctypes.data, b.ctypes.data,
                                           r.ctypes.data_as(f32p), M, N, K) == 0
        assert scaled_rel_err(r, got) <= 1e-5


def attention_f64(q, k, v, q_offset, kv_len, causal):
    rows, nq, hd = q.shape
    nkv = k.shape[1]
    out = np.zeros_like(q, dtype=np.float64)
    for h in range(nq):
        kh = k[:kv_len, h // (nq // nkv)].astype(np.float64)
        vh = v[:kv_len, h // (nq // nkv)].astype(np.float64)
        s = q[:, h].astype(np.float64) @ kh.T / np.sqrt(hd)
        if causal:
            pos = q_offset + np.arange(rows)[:, None]
            s = np.where(np.arange(kv_len)[None, :] <= pos, s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ vh
    return out


@pytest.mark.parametrize("rows,nq,nkv,hd,off,kv_len,causal", [
    (37, 8, 2, 64, 0, 37, True), (5, 28, 4, 128, 100, 105, True), (1, 2, 1, 128, 47, 48, True),
    (6, 4, 4, 32, 0, 20, False), (4, 2, 1, 128, 10, 12, True)])
def test_attention_closed_form_reference_and_invariants(rows, nq, nkv, hd, off, kv_len, causal):
    q = oracle.normal_f32((rows, nq, hd), 10)
    k = oracle.normal_f32((kv_len, nkv, hd), 11)
    v = oracle.normal_f32((kv_len, nkv, hd), 12)
    got = oracle.attention_prefill_f32(q, k, v, off, kv_len, causal)
    assert scaled_rel_err(got, attention_f64(q, k, v, off, kv_len, causal)) <= 2e-6
    if oracle.ref is not None:
        r = np.empty_like(q)
        assert oracle.ref.vv_attention_prefill_cpu(
            q.ctypes.data_as(f32p), k.ctypes.data_as(f32p), v.ctypes.data_as(f32p),
            r.ctypes.data_as(f32p), nq, nkv, hd, rows, off, kv_len, causal) == 0
        assert scaled_rel_err(r, got) <= 1e-5
    # a row's output is a convex combination of the V rows it may see
    lo, hi = v[:kv_len].min(axis=0), v[:kv_len].max(axis=0)
    g = nq // nkv
    assert (got <= np.repeat(hi, g, axis=0)[None] + 1e-5).all()
    assert (got >= np.repeat(lo, g, axis=0)[None] - 1e-5).all()
    if causal:
        # changing keys/values beyond a query's position changes nothing for it
        k2, v2 = k.copy(), v.copy()
        k2[off + 1:] += 5.0
        v2[off + 1:] -= 3.0
        again = oracle.attention_prefill_f32(q, k2, v2, off, kv_len, True)
        assert np.array_equal(again[0], got[0])
        # the decode form: the last row alone equals the last row of the batch
        last = oracle.attention_prefill_f32(q[-1:], k, v, off + rows - 1, kv_len, True)
        assert np.array_equal(last[0], got[-1])


def test_argmax_first_against_numpy_and_reference():
    """In-order scan, first maximum: numpy's argmax has the same rule; the
    compiled reference's vv_sample_greedy_cpu is the function restated."""
    rng = np.random.default_rng(3)
    cases = [rng.standard_normal(1000).astype(np.float32), np.array([-3.0], np.float32),
             np.array([1.0, 5.0, 5.0, 2.0, 5.0], np.float32), -np.ones(77, np.float32),
             np.array([-np.inf, -np.inf, -1e30], np.float32)]
    for x in cases:
        tok, val = oracle.argmax_first(x)
        assert tok == int(np.argmax(x)) and val == float(x.max())
        if oracle.ref is not None and hasattr(oracle.ref, "vv_sample_greedy_cpu"):
            t = C.c_int32()
            assert oracle.ref.vv_sample_greedy_cpu(x.ctypes.data_as(f32p), x.size, C.byref(t)) == 0
            assert t.value == tok
    nan_mid = np.array([1.0, np.nan, 3.0, np.nan, 2.0], np.float32)      # a NaN never wins once a number leads
    assert oracle.argmax_first(nan_mid)[0] == 2
