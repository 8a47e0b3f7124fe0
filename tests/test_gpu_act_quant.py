"""GPU parity tests of the int8 activation quantisers through the C ABI.

The contract is the one the reference's own test checks
(tests/test_int8_linear.c:295-354): quantising the FP16 values the UNFUSED op
wrote, on the CPU, must give exactly the bytes, scales and per-32 sums the
fused *_q8 kernel produced — for every layout, at K in {1536, 3584, 8960,
18944} and M in {1, 7, 285}. Everything here is bit-exact.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import bits_of, dev, ok, stream, to_dev

pytestmark = pytest.mark.gpu
EPS = 1e-6


def run_quant(which, d_x, d_x2, d_w, M, K, layout, with_xsum=True):
    xq = torch.zeros(M, K, dtype=torch.int8, device="cuda")
    sx = torch.zeros(M, dtype=torch.float32, device="cuda")
    xs = torch.zeros(M, K // 32, dtype=torch.int32, device="cuda")
    xs_ptr = xs.data_ptr() if with_xsum else None
    if which == "act_quant":
        ok(dev.vv_act_quant_dev(d_x.data_ptr(), M, K, layout, xq.data_ptr(), sx.data_ptr(), xs_ptr, stream()))
    elif which == "rmsnorm_q8":
        ok(dev.vv_rmsnorm_q8_dev(d_x.data_ptr(), d_w.data_ptr(), M, K, EPS, layout, xq.data_ptr(),
                                 sx.data_ptr(), xs_ptr, stream()))
    else:
        ok(dev.vv_swiglu_q8_dev(d_x.data_ptr(), d_x2.data_ptr(), M, K, layout, xq.data_ptr(),
                                sx.data_ptr(), xs_ptr, stream()))
    torch.cuda.synchronize()
    return xq.cpu().numpy(), sx.cpu().numpy(), xs.cpu().numpy()


def unfused_fp16(which, d_x, d_x2, d_w, M, K):
    """The FP16 values the unfused op writes (device), as bit patterns."""
    if which == "act_quant":
        return bits_of(d_x)
    d_y = torch.empty(M, K, dtype=torch.float16, device="cuda")
    if which == "rmsnorm_q8":
        ok(dev.vv_rmsnorm_dev(d_x.data_ptr(), d_w.data_ptr(), d_y.data_ptr(), M, K, EPS, stream()))
    else:
        ok(dev.vv_swiglu_dev(d_x.data_ptr(), d_x2.data_ptr(), d_y.data_ptr(), M * K, stream()))
    return bits_of(d_y)


@pytest.mark.parametrize("K", [1536, 3584, 8960, 18944])
@pytest.mark.parametrize("M", [1, 7, 285])
def test_quantisers_reference_shapes(M, K):
    x = oracle.normal_f16((M, K), 3 * K + M, std=4.0 / 3)
    x2 = oracle.normal_f16((M, K), 5 * K + M, std=1.0)
    w = oracle.normal_f16((K,), 7, mean=0.5, std=0.13)
    if M > 2:
        x[1] = 0                                           # a zero row: scale 0
    d_x, d_x2, d_w = to_dev(x), to_dev(x2), to_dev(w)
    for which in ("act_quant", "rmsnorm_q8", "swiglu_q8"):
        hy = unfused_fp16(which, d_x, d_x2, d_w, M, K)
        f = oracle.widen(hy)
        for layout in range(4):
            q, sx, xs = run_quant(which, d_x, d_x2, d_w, M, K, layout)
            rq, rsx, rxs = oracle.quant_act_q8(f, layout)
            what = f"{which} M={M} K={K} layout={layout}"
            assert np.array_equal(q, rq), what
            assert np.array_equal(sx.view(np.uint32), rsx.view(np.uint32)), what
            assert np.array_equal(xs, rxs), what
        # xsum is optional
        q2, sx2, xs2 = run_quant(which, d_x, d_x2, d_w, M, K, 0, with_xsum=False)
        assert not xs2.any()
        rq, rsx, _ = oracle.quant_act_q8(f, 0)
        assert np.array_equal(q2, rq) and np.array_equal(sx2, rsx)
    assert np.array_equal(bits_of(d_x), x) and np.array_equal(bits_of(d_x2), x2)   # inputs untouched


@pytest.mark.parametrize("K", [32, 256, 288, 1024, 2048, 4096, 4128, 8192, 8224, 16384, 22528])
def test_quantiser_widths_and_rounding(K):
    """Widths at the edges of the 1/2/3-chunks-per-thread ranges, and ties."""
    M = 5
    x = oracle.normal_f16((M, K), K, std=2.0)
    x[0, :] = oracle.narrow(np.full(K, 0.5, np.float32))
    x[0, 0] = oracle.narrow(np.array([127.0], np.float32))[0]     # inv = 1 exactly: 0.5 -> 0 (half to even)
    x[1, :8] = oracle.narrow(np.array([127, 1.5, 2.5, 3.5, -1.5, -2.5, 126.5, -126.5], np.float32))
    d_x = to_dev(x)
    for layout in range(4):
        q, sx, xs = run_quant("act_quant", d_x, None, None, M, K, layout)
        rq, rsx, rxs = oracle.quant_act_q8(oracle.widen(x), layout)
        assert np.array_equal(q, rq) and np.array_equal(sx, rsx) and np.array_equal(xs, rxs), (K, layout)
    q, _, _ = run_quant("act_quant", d_x, None, None, M, K, 0)
    assert q[0, 0] == 127 and not q[0, 1:].any()
    # the fused norm at the same widths (one wave per row up to 4096, workgroup per row beyond)
    if K >= 256:
        x2 = oracle.normal_f16((M, K), K + 1, std=1.5)
        w = oracle.normal_f16((K,), 9, mean=1.0, std=0.2)
        d_x2, d_w = to_dev(x2), to_dev(w)
        hy = oracle.widen(unfused_fp16("rmsnorm_q8", d_x2, None, d_w, M, K))
        for layout in range(4):
            q, sx, xs = run_quant("rmsnorm_q8", d_x2, None, d_w, M, K, layout)
            rq, rsx, rxs = oracle.quant_act_q8(hy, layout)
            assert np.array_equal(q, rq) and np.array_equal(sx, rsx) and np.array_equal(xs, rxs), (K, layout)


def test_quantiser_status_codes():
    x = torch.zeros(4, 64, dtype=torch.float16, device="cuda")
    q = torch.zeros(4, 64, dtype=torch.int8, device="cuda")
    s = torch.zeros(4, dtype=torch.float32, device="cuda")
    P, Q, S = x.data_ptr(), q.data_ptr(), s.data_ptr()
    assert dev.vv_act_quant_dev(None, 4, 64, 0, Q, S, None, None) == dev.VV_ERR_NULL_PTR
    assert dev.vv_act_quant_dev(P, 4, 64, 0, None, S, None, None) == dev.VV_ERR_NULL_PTR
    assert dev.vv_rmsnorm_q8_dev(P, None, 4, 256, EPS, 0, Q, S, None, None) == dev.VV_ERR_NULL_PTR
    assert dev.vv_swiglu_q8_dev(P, None, 4, 64, 0, Q, S, None, None) == dev.VV_ERR_NULL_PTR
    assert dev.vv_act_quant_dev(P, 0, 64, 0, Q, S, None, None) == dev.VV_ERR_INVALID_ARG
    assert dev.vv_act_quant_dev(P, 4, 64, 4, Q, S, None, None) == dev.VV_ERR_INVALID_ARG
    assert dev.vv_act_quant_dev(P, 4, 48, 0, Q, S, None, None) == dev.VV_ERR_UNSUPPORTED      # K % 32
    assert dev.vv_act_quant_dev(P, 4, 22560, 0, Q, S, None, None) == dev.VV_ERR_UNSUPPORTED   # K too wide
    assert dev.vv_rmsnorm_q8_dev(P, P, 4, 64, EPS, 0, Q, S, None, None) == dev.VV_ERR_UNSUPPORTED  # K < 256
    assert dev.vv_act_quant_dev(P + 2, 1, 64, 0, Q, S, None, None) == dev.VV_ERR_UNSUPPORTED  # unaligned
    assert dev.vv_col_absmax_dev(None, 1, 8, S, None) == dev.VV_ERR_NULL_PTR
    assert dev.vv_col_absmax_dev(P, 0, 8, S, None) == dev.VV_ERR_INVALID_ARG


def test_fused_equals_op_then_quant_at_prefill_size():
    """T = 14449: fused kernels == unfused op followed by vv_act_quant_dev, all on the
    device, bit for bit; sampled rows against the CPU quantiser."""
    T, H, I_FF = 14449, 3584, 18944
    gen = torch.Generator(device="cuda").manual_seed(8)
    x = torch.randn(T, H, generator=gen, device="cuda").half()
    w = to_dev(oracle.normal_f16((H,), 7, mean=1.0, std=0.1))
    y = torch.empty_like(x)
    ok(dev.vv_rmsnorm_dev(x.data_ptr(), w.data_ptr(), y.data_ptr(), T, H, EPS, stream()))
    for layout in (0, 2):
        fq, fsx, fxs = run_quant("rmsnorm_q8", x, None, w, T, H, layout)
        uq, usx, uxs = run_quant("act_quant", y, None, None, T, H, layout)
        assert np.array_equal(fq, uq) and np.array_equal(fsx, usx) and np.array_equal(fxs, uxs)
    rows = np.array([0, 1, 4095, 4096, 14447, 14448])
    rq, rsx, rxs = oracle.quant_act_q8(oracle.widen(bits_of(y)[rows]), 2)
    assert np.array_equal(fq[rows], rq) and np.array_equal(fsx[rows], rsx) and np.array_equal(fxs[rows], rxs)
    del x, y

    T2 = 4096
    g = (torch.randn(T2, I_FF, generator=gen, device="cuda") * 2).half()
    u = (torch.randn(T2, I_FF, generator=gen, device="cuda") * 2).half()
    o = torch.empty_like(g)
    ok(dev.vv_swiglu_dev(g.data_ptr(), u.data_ptr(), o.data_ptr(), T2 * I_FF, stream()))
    fq, fsx, fxs = run_quant("swiglu_q8", g, u, None, T2, I_FF, 3)
    uq, usx, uxs = run_quant("act_quant", o, None, None, T2, I_FF, 3)
    assert np.array_equal(fq, uq) and np.array_equal(fsx, usx) and np.array_equal(fxs, uxs)


@pytest.mark.parametrize("M,K", [(1, 3584), (70, 18944), (285, 100), (5000, 3584)])
def test_col_absmax_exact_and_accumulating(M, K):
    """tests/test_int8_linear.c:356-… : per-column absmax, accumulated over calls."""
    a = oracle.normal_f16((M, K), M + K, std=2.0)
    b = oracle.normal_f16((M, K), M + K + 1, std=0.5)
    acc = torch.zeros(K, dtype=torch.float32, device="cuda")
    d_a, d_b = to_dev(a), to_dev(b)
    ok(dev.vv_col_absmax_dev(d_a.data_ptr(), M, K, acc.data_ptr(), stream()))
    want = np.abs(oracle.widen(a)).max(axis=0)
    assert np.array_equal(acc.cpu().numpy(), want)
    ok(dev.vv_col_absmax_dev(d_b.data_ptr(), M, K, acc.data_ptr(), stream()))
    want = np.maximum(want, np.abs(oracle.widen(b)).max(axis=0))
    assert np.array_equal(acc.cpu().numpy(), want)
