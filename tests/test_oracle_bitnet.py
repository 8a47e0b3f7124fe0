"""CPU checks of the oracle's BitNet restatement (ternary and int8 integer
layers): against closed forms in numpy, and bit for bit against the reference's
own src/cpu/bitnet_cpu.c where oracle/_ref holds it compiled."""
import ctypes as C

import numpy as np
import pytest

import oracle

needs_ref = pytest.mark.skipif(oracle.ref is None or not hasattr(oracle.ref, "vv_ternary_linear_cpu"),
                               reason="oracle/_ref not built (needs the reference tree)")


def ternary(N, K, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(-1, 2, (N, K)).astype(np.int8)


def test_i2s_layout_is_the_documented_one():
    """bitnet.h:13-24: byte j of a 32-byte block holds k = j, j+32, j+64, j+96 in bits 7:6 .. 1:0; code = t + 1."""
    t = ternary(3, 256, 1)
    codes = oracle.ternary_pack(t)
    assert codes.shape == (3, 64)
    for n in range(3):
        for k in range(256):
            b, r = divmod(k, 128)
            code = (codes[n, b * 32 + r % 32] >> (6 - 2 * (r // 32))) & 3
            assert code == t[n, k] + 1
    with pytest.raises(Exception):
        oracle.ternary_pack(np.full((1, 128), 2, np.int8))


def test_activation_quantiser_closed_form():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((5, 384)) * 3).astype(np.float32)
    x[1] = 0.0                                    # amax floor 1e-5
    x[2, 7] = 1000.0
    q, s, sm = oracle.bn_act_quant(x)
    amax = np.maximum(np.abs(x).max(1).astype(np.float64), 1e-5)
    assert np.array_equal(s, (127.0 / amax).astype(np.float32))
    # the fused multiply-add never rounds x * s on its own: round_half_even of the exact product
    exact = x.astype(np.float64) * s.astype(np.float64)[:, None]
    want = np.clip(np.rint(exact), -128, 127).astype(np.int8)
    off = q != want
    # where the FP32 sum with 1.5 * 2^23 could not represent the tie exactly the two may differ by at most one step,
    # and only when the exact product sits within 2^-24 relative of a half-integer
    frac = np.abs(exact - np.floor(exact) - 0.5)
    assert np.all(frac[off] < 1e-6) and np.all(np.abs(q.astype(int) - want)[off] <= 1)
    assert np.array_equal(sm, q.astype(np.int32).sum(1))
    assert q[1].max() == 0 and q[2, 7] == 127


def test_ternary_and_int8_products_closed_form():
    rng = np.random.default_rng(3)
    M, N, K = 5, 24, 256
    t = ternary(N, K, 4)
    q = rng.integers(-128, 128, (M, K), dtype=np.int8)
    xs = rng.uniform(0.5, 40.0, M).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    acc, y = oracle.ternary_linear(q, xs, oracle.ternary_pack(t), 0.037, bias)
    want = q.astype(np.int64) @ t.astype(np.int64).T
    assert np.array_equal(acc, want.astype(np.int32))
    step = (want.astype(np.float32) / xs[:, None]) * np.float32(0.037) + bias[None, :]
    assert np.array_equal(y, step.astype(np.float32))
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    acc, y, am = oracle.i8_linear(q, 3.5, w, 0.011, bias)
    want = q.astype(np.int64) @ w.astype(np.int64).T
    assert np.array_equal(acc, want.astype(np.int32))
    d = np.float32(0.011) / np.float32(3.5)
    step = want.astype(np.float32) * d + bias[None, :]
    assert np.array_equal(y, step) and am == float(np.abs(step).max())
    rq, inv = oracle.i8s_requant(y, am, False)
    assert inv == float(np.float32(127.0) / np.float32(am))
    assert np.array_equal(rq, np.rint(np.clip(y * np.float32(inv), -127, 127)).astype(np.int8))
    relu, _ = oracle.i8s_requant(y, am, True)
    assert relu.min() == 0 and np.array_equal(relu, np.maximum(rq, 0)) and max(rq.max(), -rq.min()) == 127
    assert oracle.i8s_requant(y, 0.0, False)[1] == 0.0
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    tok, val = oracle.i8_head_argmax(q[0], 9.0, w, ws)
    logits = (want[0].astype(np.float32) * ws) / np.float32(9.0)
    assert tok == int(np.argmax(logits)) and val == float(logits.max())
    w2 = np.concatenate([w, w[tok:tok + 1]])                   # a tie goes to the lowest index
    assert oracle.i8_head_argmax(q[0], 9.0, w2, np.concatenate([ws, ws[tok:tok + 1]]))[0] == tok


@needs_ref
@pytest.mark.parametrize("M,N,K", [(1, 40, 128), (7, 33, 384), (20, 130, 2048)])
def test_against_the_compiled_reference(M, N, K):
    rng = np.random.default_rng(M + N)
    ref = oracle.ref
    t = ternary(N, K, 5)
    codes = oracle.ternary_pack(t)
    theirs = np.empty_like(codes)
    assert ref.vv_ternary_pack(t.ctypes.data, N, K, theirs.ctypes.data) == 0
    assert np.array_equal(codes, theirs)
    x = (rng.standard_normal((M, K)) * 2.5).astype(np.float32)
    x.reshape(-1)[::97] *= 30.0
    q, s, sm = oracle.bn_act_quant(x)
    q2, s2, sm2 = np.empty_like(q), np.empty_like(s), np.empty_like(sm)
    assert ref.vv_act_quant_i8_cpu(x.ctypes.data, M, K, q2.ctypes.data, s2.ctypes.data, sm2.ctypes.data) == 0
    assert np.array_equal(q, q2) and np.array_equal(s, s2) and np.array_equal(sm, sm2)
    bias = rng.standard_normal(N).astype(np.float32)
    acc, y = oracle.ternary_linear(q, s, codes, 0.0123, bias)
    acc2, y2 = np.empty_like(acc), np.empty_like(y)
    assert ref.vv_ternary_gemm_i32_cpu(q.ctypes.data, codes.ctypes.data, acc2.ctypes.data, M, N, K) == 0
    assert ref.vv_ternary_linear_cpu(q.ctypes.data, s.ctypes.data, codes.ctypes.data, 0.0123, bias.ctypes.data,
                                     y2.ctypes.data, M, N, K) == 0
    assert np.array_equal(acc, acc2) and np.array_equal(y.view(np.uint32), y2.view(np.uint32))
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    acc, y, am = oracle.i8_linear(q, 7.25, w, 0.004, bias)
    am2 = np.zeros(1, np.float32)
    assert ref.vv_i8_gemm_i32_cpu(q.ctypes.data, w.ctypes.data, acc2.ctypes.data, M, N, K) == 0
    assert ref.vv_i8_linear_cpu(q.ctypes.data, 7.25, w.ctypes.data, 0.004, bias.ctypes.data, y2.ctypes.data,
                                am2.ctypes.data, M, N, K) == 0
    assert np.array_equal(acc, acc2) and np.array_equal(y.view(np.uint32), y2.view(np.uint32)) and am == float(am2[0])
    for relu in (False, True):
        rq, inv = oracle.i8s_requant(y, am, relu)
        rq2, inv2 = np.empty_like(rq), np.zeros(1, np.float32)
        assert ref.vv_i8s_requant_cpu(y.ctypes.data, y.size, am, int(relu), rq2.ctypes.data, inv2.ctypes.data) == 0
        assert np.array_equal(rq, rq2) and inv == float(inv2[0])
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    tok, val = oracle.i8_head_argmax(q[0], float(s[0]), w, ws)
    tok2, val2 = np.zeros(1, np.int32), np.zeros(1, np.float32)
    assert ref.vv_i8_head_argmax_cpu(q[0].ctypes.data, float(s[0]), w.ctypes.data, ws.ctypes.data, N, K,
                                     tok2.ctypes.data, val2.ctypes.data) == 0
    assert tok == int(tok2[0]) and val == float(val2[0])
