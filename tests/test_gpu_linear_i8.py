"""GPU parity tests of the W8A8 linear layer through the C ABI.

The products are summed in int32 (exact) and the epilogue follows the CPU
kernel operation for operation, so the bar is bit equality: the FP32 output
against the oracle's FP32 values, the FP16 output against their
round-to-nearest-even bits, for every kernel family, tile shape and edge.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import bits_of, dev, ok, stream, to_dev

pytestmark = pytest.mark.gpu

AUTO, GEMV, MMA, SIMT = 0, 1, 2, 3


def operands(M, N, K, seed, wide=False):
    rng = np.random.default_rng(seed)
    lo = -128 if wide else -127
    xq = rng.integers(lo, 128, (M, K), dtype=np.int8)
    w = rng.integers(lo, 128, (N, K), dtype=np.int8)
    sx = (rng.random(M, dtype=np.float32) * 0.05 + 1e-3).astype(np.float32)
    sw = (rng.random(N, dtype=np.float32) * 0.01 + 1e-4).astype(np.float32)
    bias = oracle.normal_f16((N,), seed + 1, std=0.5)
    res = oracle.normal_f16((M, N), seed + 2, std=2.0)
    return xq, sx, w, sw, bias, res


def i8_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run(xq, sx, w, sw, bias=None, res=None, f32=False, path=AUTO, alias=False):
    M, K = xq.shape
    N = w.shape[0]
    d_xq, d_w, d_sx, d_sw = i8_dev(xq), i8_dev(w), i8_dev(sx), i8_dev(sw)
    d_b = to_dev(bias) if bias is not None else None
    d_r = to_dev(res) if res is not None else None
    if alias:
        d_y = d_r
    else:
        d_y = torch.full((M, N), float("nan"), dtype=torch.float32 if f32 else torch.float16, device="cuda")
    ok(dev.vv_w8a8_linear_dev(d_xq.data_ptr(), d_sx.data_ptr(), d_w.data_ptr(), d_sw.data_ptr(),
                              d_b.data_ptr() if d_b is not None else None,
                              d_r.data_ptr() if d_r is not None else None,
                              d_y.data_ptr(), 1 if f32 else 0, M, N, K, path, stream()))
    torch.cuda.synchronize()
    return d_y.cpu().numpy() if f32 else bits_of(d_y)


def same_f32(got, want, what):
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), \
        f"{what}: {(got.view(np.uint32) != want.view(np.uint32)).sum()} FP32 values differ"


SHAPES = [(1, 64, 16), (1, 3584, 3584), (1, 18944, 3584), (1, 8200, 512), (2, 100, 48), (3, 512, 3584), (5, 77, 1040),
          (8, 1000, 1536), (9, 64, 64), (16, 30, 48), (29, 512, 3584), (33, 77, 528), (64, 256, 512),
          (65, 3584, 128), (100, 130, 80), (130, 101, 208), (257, 37, 16), (285, 3584, 3584), (300, 4608, 272),
          (4100, 8200, 64),
          # K % 128 == 0 above 64 rows: the copy-fed 256x256 tiles with the last rows split off, the 128x128 tile
          # with two and with four stages (the 64x64 one: 65 and 285 rows above)
          (4100, 8200, 128), (2100, 2100, 256), (1100, 2048, 128)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_w8a8_bit_exact_against_oracle(M, N, K):
    xq, sx, w, sw, bias, res = operands(M, N, K, 7 * M + N)
    want32, want16 = oracle.w8a8_linear(xq, sx, w, sw, bias, res)
    same_f32(run(xq, sx, w, sw, bias, res, f32=True), want32, f"f32 {M}x{N}x{K}")
    assert np.array_equal(run(xq, sx, w, sw, bias, res), want16), f"f16 {M}x{N}x{K}"
    plain32, plain16 = oracle.w8a8_linear(xq, sx, w, sw)
    same_f32(run(xq, sx, w, sw, f32=True), plain32, f"f32 plain {M}x{N}x{K}")
    assert np.array_equal(run(xq, sx, w, sw), plain16), f"f16 plain {M}x{N}x{K}"


@pytest.mark.parametrize("M,N,K", [(1, 96, 64), (4, 260, 128), (8, 3584, 512), (40, 100, 64), (200, 264, 144)])
@pytest.mark.parametrize("with_bias,with_res", [(True, False), (False, True)])
def test_w8a8_bias_or_residual_alone(M, N, K, with_bias, with_res):
    xq, sx, w, sw, bias, res = operands(M, N, K, 31 + M)
    b, r = (bias if with_bias else None), (res if with_res else None)
    want32, want16 = oracle.w8a8_linear(xq, sx, w, sw, b, r)
    same_f32(run(xq, sx, w, sw, b, r, f32=True), want32, "f32")
    assert np.array_equal(run(xq, sx, w, sw, b, r), want16)


@pytest.mark.parametrize("M,N,K", [(1, 512, 256), (7, 130, 64), (64, 512, 256), (300, 264, 128)])
def test_w8a8_residual_may_alias_output(M, N, K):
    """y += result: the residual buffer is the output buffer."""
    xq, sx, w, sw, bias, res = operands(M, N, K, 91 + M)
    _, want16 = oracle.w8a8_linear(xq, sx, w, sw, bias, res)
    assert np.array_equal(run(xq, sx, w, sw, bias, res, alias=True), want16)


@pytest.mark.parametrize("M,N,K", [(1, 300, 512), (3, 8200, 256), (8, 16400, 64), (8, 77, 48)])
def test_w8a8_kernel_families_agree(M, N, K):
    """Up to eight rows both families serve the shape, with the same bits."""
    xq, sx, w, sw, bias, res = operands(M, N, K, 17 + N)
    want32, _ = oracle.w8a8_linear(xq, sx, w, sw, bias, res)
    for path in (AUTO, GEMV, MMA, SIMT):
        same_f32(run(xq, sx, w, sw, bias, res, f32=True, path=path), want32, f"path {path}")


def test_w8a8_extreme_values_do_not_saturate():
    """-128 * -128 over the longest K of the model: 3.1e8, inside int32."""
    M, N, K = 9, 64, 18944
    xq = np.full((M, K), -128, np.int8)
    w = np.full((N, K), -128, np.int8)
    w[1::2] = 127
    sx, sw = np.full(M, 2.0 ** -10, np.float32), np.full(N, 2.0 ** -12, np.float32)
    want32, _ = oracle.w8a8_linear(xq, sx, w, sw)
    assert want32[0, 0] == np.float32(128 * 128 * K) * np.float32(2.0 ** -22)
    same_f32(run(xq, sx, w, sw, f32=True), want32, "mfma")
    same_f32(run(xq[:4], sx[:4], w, sw, f32=True), want32[:4], "gemv")


def test_w8a8_unaligned_vectors_and_ragged_n():
    """bias / scale / output pointers that are only element-aligned, N % 4 != 0."""
    M, N, K = 37, 103, 96
    xq, sx, w, sw, bias, res = operands(M, N, K, 5)
    want32, want16 = oracle.w8a8_linear(xq, sx, w, sw, bias, res)
    same_f32(run(xq, sx, w, sw, bias, res, f32=True), want32, "ragged N")
    # N % 4 == 0 but every FP16 / FP32 operand one element off a 16-byte boundary
    N = 104
    xq, sx, w, sw, bias, res = operands(M, N, K, 6)
    want32, want16 = oracle.w8a8_linear(xq, sx, w, sw, bias, res)
    d_xq, d_w, d_sx = i8_dev(xq), i8_dev(w), i8_dev(sx)
    pad = lambda t: torch.cat([torch.zeros(1, dtype=t.dtype, device="cuda"), t.reshape(-1)])[1:]
    d_sw, d_b, d_r = pad(i8_dev(sw)), pad(to_dev(bias)), pad(to_dev(res))
    d_y = pad(torch.zeros(M * N, dtype=torch.float16, device="cuda"))
    assert d_sw.data_ptr() % 16 != 0 and d_b.data_ptr() % 8 != 0 and d_y.data_ptr() % 8 != 0
    ok(dev.vv_w8a8_linear_dev(d_xq.data_ptr(), d_sx.data_ptr(), d_w.data_ptr(), d_sw.data_ptr(), d_b.data_ptr(),
                              d_r.data_ptr(), d_y.data_ptr(), 0, M, N, K, AUTO, stream()))
    assert np.array_equal(bits_of(d_y).reshape(M, N), want16)


def test_w8a8_follows_the_device_quantiser():
    """FP16 activations -> vv_act_quant_dev -> vv_w8a8_linear_dev equals the
    oracle's quantiser followed by the oracle's linear, and is close to the
    unquantised product."""
    M, N, K = 70, 512, 3584
    x = oracle.normal_f16((M, K), 3)
    wf = oracle.normal_f32((N, K), 4, std=K ** -0.5)
    sw = (np.abs(wf).max(axis=1) / 127.0).astype(np.float32)
    w = np.clip(np.rint(wf / sw[:, None]), -127, 127).astype(np.int8)
    d_x, d_w, d_sw = to_dev(x), i8_dev(w), i8_dev(sw)
    d_xq = torch.empty((M, K), dtype=torch.int8, device="cuda")
    d_sx = torch.empty(M, dtype=torch.float32, device="cuda")
    d_y = torch.empty((M, N), dtype=torch.float32, device="cuda")
    ok(dev.vv_act_quant_dev(d_x.data_ptr(), M, K, 0, d_xq.data_ptr(), d_sx.data_ptr(), None, stream()))
    ok(dev.vv_w8a8_linear_dev(d_xq.data_ptr(), d_sx.data_ptr(), d_w.data_ptr(), d_sw.data_ptr(), None, None,
                              d_y.data_ptr(), 1, M, N, K, AUTO, stream()))
    torch.cuda.synchronize()
    xq, sx, _ = oracle.quant_act_q8(oracle.widen(x), 0, want_xsum=False)
    want32, _ = oracle.w8a8_linear(xq, sx, w, sw)
    same_f32(d_y.cpu().numpy(), want32, "quantise + linear")
    dense = oracle.widen(x).astype(np.float64) @ wf.astype(np.float64).T
    assert np.max(np.abs(want32 - dense)) / np.max(np.abs(dense)) < 0.03


def test_w8a8_prefill_shape_sampled_rows():
    """The model's prefill shape (T = 14449 rows through a 3584 x 3584
    projection): 48 sampled rows against the oracle, and the whole output
    against the same call split in two row blocks (rows are independent)."""
    M, N, K = 14449, 3584, 3584
    xq, sx, w, sw, bias, _ = operands(M, N, K, 11)
    d_xq, d_w, d_sx, d_sw, d_b = i8_dev(xq), i8_dev(w), i8_dev(sx), i8_dev(sw), to_dev(bias)
    d_y = torch.empty((M, N), dtype=torch.float16, device="cuda")
    args = lambda r0, rows: (d_xq[r0:].data_ptr(), d_sx[r0:].data_ptr(), d_w.data_ptr(), d_sw.data_ptr(),
                             d_b.data_ptr(), None)
    ok(dev.vv_w8a8_linear_dev(*args(0, M), d_y.data_ptr(), 0, M, N, K, AUTO, stream()))
    got = bits_of(d_y)
    rows = np.sort(np.random.default_rng(1).choice(M, 48, replace=False))
    rows[0], rows[-1] = 0, M - 1
    _, want16 = oracle.w8a8_linear(xq[rows], sx[rows], w, sw, bias)
    assert np.array_equal(got[rows], want16)
    d_z = torch.empty((M, N), dtype=torch.float16, device="cuda")
    cut = 6000
    ok(dev.vv_w8a8_linear_dev(*args(0, cut), d_z.data_ptr(), 0, cut, N, K, AUTO, stream()))
    ok(dev.vv_w8a8_linear_dev(*args(cut, M - cut), d_z[cut:].data_ptr(), 0, M - cut, N, K, AUTO, stream()))
    assert np.array_equal(bits_of(d_z), got)


@pytest.mark.parametrize("M", [1, 6, 40])
def test_i8_linear_multi_equals_single_calls(M):
    K = 512
    Ns = [512, 128, 136]
    xq, sx, *_ = operands(M, 8, K, 50 + M)
    d_xq, d_sx = i8_dev(xq), i8_dev(sx)
    keep, projs, wants = [], (dev.I8Proj * 3)(), []
    for i, N in enumerate(Ns):
        _, _, w, sw, bias, _ = operands(M, N, K, 60 + i)
        b = bias if i != 1 else None
        d_w, d_sw = i8_dev(w), i8_dev(sw)
        d_b = to_dev(b) if b is not None else None
        d_y = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        keep.append((d_w, d_sw, d_b, d_y))
        projs[i] = dev.I8Proj(d_w.data_ptr(), d_sw.data_ptr(), None, d_b.data_ptr() if d_b is not None else None,
                          d_y.data_ptr(), N)
        wants.append(oracle.w8a8_linear(xq, sx, w, sw, b)[1])
    call = lambda layout, w4, n: dev.vv_i8_linear_multi_dev(d_xq.data_ptr(), layout, d_sx.data_ptr(), None, w4,
                                                            C.addressof(projs), n, 0, M, K, stream())
    ok(call(0, 0, 3))
    for (_, _, _, d_y), want in zip(keep, wants):
        assert np.array_equal(bits_of(d_y), want)
    assert call(1, 0, 3) == dev.VV_ERR_UNSUPPORTED       # W8A8 reads column order only
    assert call(0, 0, 0) == dev.VV_ERR_INVALID_ARG
    assert dev.vv_i8_linear_multi_dev(None, 0, d_sx.data_ptr(), None, 0, C.addressof(projs), 3, 0, M, K,
                                      stream()) == dev.VV_ERR_NULL_PTR


def test_w8a8_argument_checks_launch_nothing():
    M, N, K = 4, 64, 64
    xq, sx, w, sw, *_ = operands(M, N, K, 1)
    d_xq, d_w, d_sx, d_sw = i8_dev(xq), i8_dev(w), i8_dev(sx), i8_dev(sw)
    d_y = torch.full((16, N), 7.0, dtype=torch.float16, device="cuda")
    X, S, W, SW, Y = d_xq.data_ptr(), d_sx.data_ptr(), d_w.data_ptr(), d_sw.data_ptr(), d_y.data_ptr()
    f = dev.vv_w8a8_linear_dev
    for args in [(None, S, W, SW), (X, None, W, SW), (X, S, None, SW), (X, S, W, None)]:
        assert f(*args, None, None, Y, 0, M, N, K, AUTO, stream()) == dev.VV_ERR_NULL_PTR
    assert f(X, S, W, SW, None, None, None, 0, M, N, K, AUTO, stream()) == dev.VV_ERR_NULL_PTR
    for m, n, k in [(0, N, K), (M, 0, K), (M, N, 0), (-1, N, K)]:
        assert f(X, S, W, SW, None, None, Y, 0, m, n, k, AUTO, stream()) == dev.VV_ERR_INVALID_ARG
    assert f(X, S, W, SW, None, None, Y, 0, M, N, K, 4, stream()) == dev.VV_ERR_INVALID_ARG
    assert f(X, S, W, SW, None, None, Y, 0, M, N, 40, AUTO, stream()) == dev.VV_ERR_UNSUPPORTED   # K % 16
    assert f(X + 4, S, W, SW, None, None, Y, 0, 1, N, 48, AUTO, stream()) == dev.VV_ERR_UNSUPPORTED
    assert f(X, S, W, SW, None, None, Y, 0, 9, N, K, GEMV, stream()) == dev.VV_ERR_UNSUPPORTED
    torch.cuda.synchronize()
    assert (d_y == 7.0).all()


# ── W4A8 ────────────────────────────────────────────────────────────────────

L_GEMV, L_MMA = 2, 3        # VV_Q8_W4_GEMV, VV_Q8_W4_MMA


def w4_problem(M, N, K, G, seed, unit=False):
    """Activations quantised by the oracle in column order and in both
    accelerator orders; codes, FP16 group scales and zero points; the codes in
    the accelerator layout with their half2 {scale, zero} table."""
    rng = np.random.default_rng(seed)
    x = rng.normal(size=(M, K)).astype(np.float32) * 3
    xq, sx, xs = oracle.quant_act_q8(x, 0)
    orders = {lay: oracle.quant_act_q8(x, lay, want_xsum=False)[0] for lay in (L_GEMV, L_MMA)}
    packed = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    zeros = rng.integers(0, 16, (N, K // G), dtype=np.uint8)
    if unit:
        scales = np.full((N, K // G), 0x3C00, np.uint16)
        sx = np.ones(M, np.float32)
    else:
        scales = rng.uniform(0.002, 0.022, (N, K // G)).astype(np.float16).view(np.uint16)
    gpu, sz = oracle.int4g_to_gpu_layout(packed, scales, zeros, G)
    bias = oracle.normal_f16((N,), seed + 1, std=0.5)
    res = oracle.normal_f16((M, N), seed + 2, std=2.0)
    return dict(xq=xq, sx=sx, xs=xs, orders=orders, packed=packed, scales=scales, zeros=zeros, gpu=gpu, sz=sz,
                bias=bias, res=res, G=G)


def run_w4(p, layout, bias=False, res=False, f32=False, path=AUTO, alias=False, expect=None, xsum=False):
    M, K = p["xq"].shape
    N = p["packed"].shape[0]
    d_xq, d_sx = i8_dev(p["orders"].get(layout, p["xq"])), i8_dev(p["sx"])
    d_w, d_sz = i8_dev(p["gpu"]), i8_dev(p["sz"])
    d_b = to_dev(p["bias"]) if bias else None
    d_r = to_dev(p["res"]) if res else None
    d_xs = i8_dev(p["xs"]) if xsum else None
    if alias:
        d_y = d_r
    else:
        d_y = torch.full((M, N), float("nan"), dtype=torch.float32 if f32 else torch.float16, device="cuda")
    st = dev.vv_w4a8_linear_dev(d_xq.data_ptr(), layout, d_sx.data_ptr(), d_xs.data_ptr() if xsum else None,
                                d_w.data_ptr(), d_sz.data_ptr(),
                                p["G"], d_b.data_ptr() if bias else None, d_r.data_ptr() if res else None,
                                d_y.data_ptr(), 1 if f32 else 0, M, N, K, path, stream())
    if expect is not None:
        assert st == expect, st
        return None
    ok(st)
    torch.cuda.synchronize()
    return d_y.cpu().numpy() if f32 else bits_of(d_y)


def want_w4(p, bias=False, res=False):
    return oracle.w4a8_linear(p["xq"], p["sx"], p["packed"], p["scales"], p["zeros"], p["G"],
                              p["bias"] if bias else None, p["res"] if res else None)


W4_SHAPES = [(1, 64, 32, 32), (3, 50, 192, 96), (1, 40, 8192, 4096), (8, 37, 18944, 32), (1, 18944, 3584, 128), (1, 3584, 3584, 128), (1, 512, 18944, 128), (2, 77, 256, 256), (5, 136, 640, 32),
             (8, 300, 640, 64), (8, 64, 1024, 512), (9, 64, 64, 32), (16, 30, 96, 32), (17, 77, 256, 256),
             (33, 136, 640, 32), (64, 300, 640, 64), (65, 64, 1024, 512), (100, 130, 160, 32), (130, 101, 224, 32),
             (285, 3584, 3584, 128), (300, 4608, 1536, 128), (921, 512, 3584, 128),
             # at most 64 rows in the MMA order with groups of 64, 128, 256: the streamed kernel, whole and partial
             # rounds of eight groups, ragged N
             (9, 100, 1152, 128), (29, 3584, 3584, 128), (28, 520, 18944, 128), (33, 77, 1280, 64),
             (64, 136, 2304, 256), (40, 4608, 1536, 128), (32, 31, 64, 64), (5, 33, 8192, 128),
             # five to eight rows: the streamed kernel reads the GEMV's order of the activations as well
             (8, 3584, 3584, 128), (7, 100, 1152, 128), (6, 520, 2304, 256), (5, 77, 1280, 64)]


@pytest.mark.parametrize("M,N,K,G", W4_SHAPES)
def test_w4a8_bit_exact_against_oracle(M, N, K, G):
    """Both kernel families (the GEMV where it serves the shape) give the
    oracle's FP32 bits and their correctly rounded FP16."""
    p = w4_problem(M, N, K, G, 3 * M + N)
    want32, want16 = want_w4(p, True, True)
    plain32, _ = want_w4(p)
    layouts = (L_GEMV, L_MMA) if M <= 8 else (L_MMA,)
    for lay in layouts:
        same_f32(run_w4(p, lay, True, True, f32=True), want32, f"f32 layout {lay}")
        assert np.array_equal(run_w4(p, lay, True, True), want16), f"f16 layout {lay}"
        same_f32(run_w4(p, lay, f32=True), plain32, f"f32 plain layout {lay}")
        same_f32(run_w4(p, lay, True, True, f32=True, xsum=True), want32, f"f32 layout {lay} with xsum")
        if lay == L_MMA and M <= 64:     # asked for by name, the LDS-tiled kernel serves these rows too
            same_f32(run_w4(p, lay, True, True, f32=True, path=MMA), want32, "f32 tiled")
        if lay == L_GEMV and M > 4:      # and the GEMV beyond the four rows AUTO gives it
            same_f32(run_w4(p, lay, True, True, f32=True, path=GEMV), want32, "f32 gemv by name")
            same_f32(run_w4(p, lay, True, True, f32=True, path=GEMV, xsum=True), want32, "f32 gemv by name, xsum")


@pytest.mark.parametrize("M,N,K,G", [(1, 256, 3584, 128), (7, 300, 640, 64), (40, 136, 640, 32), (300, 264, 1024, 512)])
def test_w4a8_unit_scales_give_the_exact_integer(M, N, K, G):
    """With every scale 1 the FP32 output is sum_k (q - z) x itself."""
    p = w4_problem(M, N, K, G, 70 + M, unit=True)
    codes = np.empty((N, K), np.int64)
    codes[:, 0::2], codes[:, 1::2] = p["packed"] >> 4, p["packed"] & 15
    codes -= np.repeat(p["zeros"].astype(np.int64), G, axis=1)
    exact = p["xq"].astype(np.int64) @ codes.T
    assert np.abs(exact).max() < 2 ** 24
    for lay in ((L_GEMV, L_MMA) if M <= 8 else (L_MMA,)):
        assert np.array_equal(run_w4(p, lay, f32=True).astype(np.int64), exact)


@pytest.mark.parametrize("M,layout", [(3, L_GEMV), (3, L_MMA), (200, L_MMA)])
def test_w4a8_residual_may_alias_output(M, layout):
    p = w4_problem(M, 264, 512, 128, 40 + M)
    _, want16 = want_w4(p, True, True)
    assert np.array_equal(run_w4(p, layout, True, True, alias=True), want16)


def test_w4a8_paths_and_layouts():
    """AUTO follows the layout; a family asked for with the other family's
    layout, or the GEMV beyond eight rows, declines."""
    p = w4_problem(4, 96, 256, 64, 9)
    want32, _ = want_w4(p)
    same_f32(run_w4(p, L_GEMV, f32=True, path=GEMV), want32, "gemv")
    for path in (MMA, SIMT):
        same_f32(run_w4(p, L_MMA, f32=True, path=path), want32, f"path {path}")
        run_w4(p, L_GEMV, path=path, expect=dev.VV_ERR_UNSUPPORTED)
    run_w4(p, L_MMA, path=GEMV, expect=dev.VV_ERR_UNSUPPORTED)
    run_w4(p, 0, expect=dev.VV_ERR_INVALID_ARG)
    run_w4(p, 1, expect=dev.VV_ERR_INVALID_ARG)
    run_w4(p, L_MMA, path=4, expect=dev.VV_ERR_INVALID_ARG)
    big = w4_problem(9, 64, 64, 32, 10)
    run_w4(big, L_GEMV, expect=dev.VV_ERR_UNSUPPORTED)
    bad_group = dict(p, G=48)
    run_w4(bad_group, L_MMA, expect=dev.VV_ERR_UNSUPPORTED)
    assert dev.vv_w4a8_linear_dev(None, L_MMA, None, None, None, None, 64, None, None, None, 0, 4, 96, 256, 0,
                                  stream()) == dev.VV_ERR_NULL_PTR


def test_w4a8_follows_the_device_quantiser():
    """vv_act_quant_dev in each accelerator order feeds the kernel that reads it."""
    M, N, K, G = 6, 512, 3584, 128
    p = w4_problem(M, N, K, G, 21)
    x = oracle.normal_f16((M, K), 5, std=2.0)
    xq, sx, _ = oracle.quant_act_q8(oracle.widen(x), 0, want_xsum=False)
    want32, _ = oracle.w4a8_linear(xq, sx, p["packed"], p["scales"], p["zeros"], G)
    d_x, d_w, d_sz = to_dev(x), i8_dev(p["gpu"]), i8_dev(p["sz"])
    for lay in (L_GEMV, L_MMA):
        d_xq = torch.empty((M, K), dtype=torch.int8, device="cuda")
        d_sx = torch.empty(M, dtype=torch.float32, device="cuda")
        d_xs = torch.empty((M, K // 32), dtype=torch.int32, device="cuda")
        d_y = torch.empty((M, N), dtype=torch.float32, device="cuda")
        ok(dev.vv_act_quant_dev(d_x.data_ptr(), M, K, lay, d_xq.data_ptr(), d_sx.data_ptr(), d_xs.data_ptr(),
                                stream()))
        ok(dev.vv_w4a8_linear_dev(d_xq.data_ptr(), lay, d_sx.data_ptr(), d_xs.data_ptr(), d_w.data_ptr(),
                                  d_sz.data_ptr(), G, None, None, d_y.data_ptr(), 1, M, N, K, AUTO, stream()))
        torch.cuda.synchronize()
        same_f32(d_y.cpu().numpy(), want32, f"layout {lay}")


@pytest.mark.parametrize("M,layout", [(6, L_GEMV), (29, L_MMA)])
def test_w4a8_streamed_rows_replay_from_a_graph(M, layout):
    """Quantiser + W4A8 layer at the row counts of the streamed kernel, captured once (the kernel's first use may
    fall inside the capture) and replayed on new activations, the program's own work in between: every replay
    gives the oracle's bits."""
    N, K, G = 2080, 3584, 128
    p = w4_problem(M, N, K, G, 23)
    d_w, d_sz = i8_dev(p["gpu"]), i8_dev(p["sz"])
    d_x = torch.zeros((M, K), dtype=torch.float16, device="cuda")
    d_xq = torch.empty((M, K), dtype=torch.int8, device="cuda")
    d_sx = torch.empty(M, dtype=torch.float32, device="cuda")
    d_xs = torch.empty((M, K // 32), dtype=torch.int32, device="cuda")
    d_y = torch.empty((M, N), dtype=torch.float32, device="cuda")
    s = C.c_void_p()
    assert dev.vv_dev_stream_create(C.byref(s)) == dev.VV_OK
    st = s.value
    torch.cuda.synchronize()
    assert dev.vv_dev_graph_begin(st) == dev.VV_OK
    ok(dev.vv_act_quant_dev(d_x.data_ptr(), M, K, layout, d_xq.data_ptr(), d_sx.data_ptr(), d_xs.data_ptr(), st))
    ok(dev.vv_w4a8_linear_dev(d_xq.data_ptr(), layout, d_sx.data_ptr(), d_xs.data_ptr(), d_w.data_ptr(),
                              d_sz.data_ptr(), G, None, None, d_y.data_ptr(), 1, M, N, K, AUTO, st))
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(st, C.byref(g)) == dev.VV_OK and g.value
    for i in range(3):
        x = oracle.normal_f16((M, K), 30 + i, std=1.0 + i)
        d_x.copy_(torch.from_numpy(x.view(np.float16)))
        torch.cuda.synchronize()
        assert dev.vv_dev_graph_launch(g.value, st) == dev.VV_OK
        assert dev.vv_dev_stream_sync(st) == dev.VV_OK
        xq, sx, _ = oracle.quant_act_q8(oracle.widen(x), 0, want_xsum=False)
        want32, _ = oracle.w4a8_linear(xq, sx, p["packed"], p["scales"], p["zeros"], G)
        same_f32(d_y.cpu().numpy(), want32, f"replay {i}")
    dev.vv_dev_graph_destroy(g.value)
    dev.vv_dev_stream_destroy(st)


@pytest.mark.parametrize("M,layout", [(2, L_GEMV), (40, L_MMA), (7, L_GEMV), (6, L_GEMV)])
def test_i8_linear_multi_w4(M, layout):
    """One launch for all projections or one call each (M = 6: wide projections of
    more than four rows go one by one), the same bits."""
    K, G = 512, 128
    sizes = (9000, 8000, 136) if M == 6 else (512, 128, 136)
    base = w4_problem(M, 8, K, G, 80 + M)
    d_xq, d_sx = i8_dev(base["orders"][layout]), i8_dev(base["sx"])
    keep, projs, wants = [], (dev.I8Proj * 3)(), []
    for i, N in enumerate(sizes):
        p = w4_problem(M, N, K, G, 90 + i)
        d_w, d_sz = i8_dev(p["gpu"]), i8_dev(p["sz"])
        d_b = to_dev(p["bias"]) if i != 1 else None
        d_y = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        keep.append((d_w, d_sz, d_b, d_y))
        projs[i] = dev.I8Proj(d_w.data_ptr(), None, d_sz.data_ptr(), d_b.data_ptr() if d_b is not None else None,
                              d_y.data_ptr(), N)
        wants.append(oracle.w4a8_linear(base["xq"], base["sx"], p["packed"], p["scales"], p["zeros"], G,
                                        p["bias"] if i != 1 else None)[1])
    ok(dev.vv_i8_linear_multi_dev(d_xq.data_ptr(), layout, d_sx.data_ptr(), None, 1, C.addressof(projs), 3, G,
                                  M, K, stream()))
    for (_, _, _, d_y), want in zip(keep, wants):
        assert np.array_equal(bits_of(d_y), want)
