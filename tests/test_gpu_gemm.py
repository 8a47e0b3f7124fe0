"""GPU parity tests of the dense FP16 GEMM (C = alpha * A * B^T + beta * C)
through the C ABI, against the oracle's double-accumulated product.

Bars: the stated one for FP16 outputs (scaled error <= 2e-3) and an
elementwise one of our own: half an FP16 ulp of the exact value plus 1e-5 of
sum_k |a||b| (FP32 accumulation over K <= 18944 stays well inside that).
Bit-exact: every tile shape against the 128x128 tile (same K order; above 64
rows, where the tile kernels run) except the tiles on the 16x16x32
instructions, which are held to it within the FP32 summation order and to
themselves bit for bit; beta = 0 never reading C, M <= 0 / N <= 0 launching nothing.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import FP16_TOL, bits_of, dev, ok, stream, to_dev
from conftest import scaled_rel_err

pytestmark = pytest.mark.gpu


def exact(a_bits, b_bits, c_bits, alpha, beta):
    a = oracle.widen(a_bits)
    ref = alpha * oracle.gemm_f16w(a, b_bits).astype(np.float64)
    if beta != 0.0:
        ref = ref + beta * oracle.widen(c_bits).astype(np.float64)
    mag = abs(alpha) * (np.abs(a).astype(np.float64) @ np.abs(oracle.widen(b_bits)).astype(np.float64).T)
    return ref, mag


def check(got_bits, ref, mag, what):
    got = oracle.widen(got_bits).astype(np.float64)
    err = scaled_rel_err(got, ref)
    assert err <= FP16_TOL, f"{what}: scaled error {err:.3e}"
    with np.errstate(over="ignore"):
        ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    bound = 0.5 * ulp + 1e-5 * mag + 2.0 ** -25
    worst = float(np.max(np.abs(got - ref) / bound))
    assert worst <= 1.0, f"{what}: {worst:.3f}x the elementwise bound"


def run(fn, d_a, d_b, d_c, M, N, K, alpha=1.0, beta=0.0):
    ok(fn(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr(), M, N, K, alpha, beta, stream()))
    return bits_of(d_c)


SHAPES = [(1, 64, 64), (2, 48, 32), (16, 30, 40), (17, 100, 264), (33, 77, 520), (49, 16, 1024), (64, 3584, 3584), (1, 3584, 3584), (3, 512, 3584), (8, 1000, 1536), (9, 64, 64),
          (29, 3584, 3584), (29, 512, 3584), (33, 4608, 1536), (64, 256, 512), (100, 128, 72),
          (285, 3584, 3584), (130, 101, 200), (257, 37, 8), (48, 512, 256), (70, 3584, 18944), (29, 18944, 512),
          (4100, 8200, 72), (4097, 8192, 64),     # enough 256x256 workgroups for the eight-wave tile
          (4100, 8200, 192), (4097, 8192, 128), (4100, 8200, 96),
          # 256x256 tiles in 4 x 8 blocks dealt to the eight XCDs: 18 and 128 whole blocks with ragged edges, no whole
          # block at all (7 tile columns), whole blocks only
          (2048, 18944, 64), (2300, 16400, 128), (19000, 1792, 64), (4096, 8192, 64),
          # the 128x128 tile fed the same way: 17 x 17, 9 x 32 and 113 x 4 tiles
          (2100, 2100, 192), (1100, 4096, 64), (14449, 512, 128), (70, 33000, 64),      # ... and one row of 258 tiles
          # the 64x64 tile fed the same way: 256 tiles or fewer (eight stages), more (four), ragged, one slab
          (2048, 512, 3584), (285, 3584, 3584), (130, 200, 64), (1000, 1100, 192), (65, 64, 128),
          # 17 .. 64 rows, K in whole 64-K lines: the weight-streaming kernel that fetches the activations by whole cache
          # lines (two, three and four row tiles; ragged N; one line; five lines, so that three waves have none; a long K)
          (17, 100, 320), (33, 52, 64), (40, 3584, 18944), (64, 3584, 1088), (48, 30, 4096), (20, 3584, 3584),
          (2, 264, 3584), (5, 3584, 18944), (16, 18944, 3584), (13, 50, 64),
          # 17 .. 64 rows, N too wide for that kernel: one row of 128x128 tiles (and just below their bar: 64-wide ones)
          (24, 18944, 3584), (64, 16300, 128), (33, 16200, 128), (17, 12800, 64), (48, 13000, 448), (32, 12900, 72),
          # one row, few long weight rows: two output columns per wave (an odd count leaves the last wave one)
          (1, 3584, 18944), (1, 37, 8192), (1, 1, 8200)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_gemm_against_oracle_and_tile(M, N, K):
    a = oracle.normal_f16((M, K), 100 + M)
    b = oracle.normal_f16((N, K), 200 + N, std=K ** -0.5)
    d_a, d_b = to_dev(a), to_dev(b)
    d_c = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    got = run(dev.vv_gemm_fp16_dev, d_a, d_b, d_c, M, N, K)     # beta = 0 over NaNs
    ref, mag = exact(a, b, None, 1.0, 0.0)
    check(got, ref, mag, f"gemm {M}x{N}x{K}")
    d_t = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    tile = run(dev.vv_gemm_fp16_tile_dev, d_a, d_b, d_t, M, N, K)
    check(tile, ref, mag, f"tile {M}x{N}x{K}")
    big = K % 64 == 0 and (M > 64 or (M > 16 and N >= 12800))      # the latter: too wide for the weight-streaming kernel
    if big:
        # the tiles fed in 128-byte slabs (the choice above 64 rows when K % 64 == 0) and the kernel that streams 128
        # columns a workgroup (17 .. 64 rows where N is very wide) multiply with the 16x16x32
        # instructions, which add 32 products at a time where the other tiles add 16: same sums, another
        # rounding of the FP32 partials
        diff = np.abs(oracle.widen(got) - oracle.widen(tile))
        assert np.all(diff <= 2.0 ** -9 * mag + 2.0 ** -14), "tile shapes must agree to FP32 summation order"
        again = run(dev.vv_gemm_fp16_dev, d_a, d_b, torch.zeros_like(d_c), M, N, K)
        assert np.array_equal(got, again), "the same call must give the same bits"
    elif M > 64 or (M > 16 and N >= 12800):   # elsewhere the weight-streaming kernel adds K in another order
        assert np.array_equal(got, tile), "tile shapes must agree bit for bit"


@pytest.mark.parametrize("M,N,K", [(1, 256, 512), (5, 100, 64), (29, 256, 512), (200, 264, 136)])
@pytest.mark.parametrize("alpha,beta", [(1.0, 1.0), (0.5, -2.0), (-1.25, 0.0)])
def test_gemm_alpha_beta(M, N, K, alpha, beta):
    a = oracle.normal_f16((M, K), 1)
    b = oracle.normal_f16((N, K), 2, std=K ** -0.5)
    c = oracle.normal_f16((M, N), 3)
    ref, mag = exact(a, b, c, alpha, beta)
    mag = mag + abs(beta) * np.abs(oracle.widen(c))
    for fn in (dev.vv_gemm_fp16_dev, dev.vv_gemm_fp16_tile_dev):
        got = run(fn, to_dev(a), to_dev(b), to_dev(c), M, N, K, alpha, beta)
        check(got, ref, mag, f"alpha {alpha} beta {beta}")


@pytest.mark.parametrize("M,N,K", [(3, 40, 131), (20, 33, 7), (70, 130, 100)])
def test_gemm_scalar_path(M, N, K):
    """K % 8 != 0, and operands that start 2 bytes off a 16-byte boundary."""
    a = oracle.normal_f16((M, K), 4)
    b = oracle.normal_f16((N, K), 5, std=K ** -0.5)
    ref, mag = exact(a, b, None, 1.0, 0.0)
    d_c = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    check(run(dev.vv_gemm_fp16_dev, to_dev(a), to_dev(b), d_c, M, N, K), ref, mag, "odd K")
    pad = torch.zeros(M * K + 1, dtype=torch.float16, device="cuda")
    pad[1:] = to_dev(a).reshape(-1)
    d_c.zero_()
    ok(dev.vv_gemm_fp16_dev(pad.data_ptr() + 2, to_dev(b).data_ptr(), d_c.data_ptr(), M, N, K,
                            1.0, 0.0, stream()))
    check(bits_of(d_c), ref, mag, "misaligned A")


def test_gemm_edges():
    d = torch.ones(64, dtype=torch.float16, device="cuda")
    p = d.data_ptr()
    assert dev.vv_gemm_fp16_dev(None, p, p, 1, 1, 8, 1.0, 0.0, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_gemm_fp16_dev(p, p, p, 0, 8, 8, 1.0, 0.0, stream()) == dev.VV_OK
    assert dev.vv_gemm_fp16_tile_dev(p, p, p, 4, 0, 8, 1.0, 0.0, stream()) == dev.VV_OK
    assert bits_of(d).tolist() == [0x3C00] * 64
    # K == 0: C = beta * C
    c = to_dev(oracle.normal_f16((2, 8), 9))
    want = (2.0 * oracle.widen(bits_of(c))).astype(np.float16).view(np.uint16)
    ok(dev.vv_gemm_fp16_dev(p, p, c.data_ptr(), 2, 8, 0, 1.0, 2.0, stream()))
    assert np.array_equal(bits_of(c), want)
    # the same at shapes that would otherwise run the 128- and 256-wide tile kernels: no operand is read
    for fn, M, N in ((dev.vv_gemm_fp16_dev, 300, 512), (dev.vv_gemm_fp16_dev, 1024, 2048),
                     (dev.vv_gemm_fp16_tile_dev, 300, 512)):
        c = to_dev(oracle.normal_f16((M, N), 10))
        want = (2.0 * oracle.widen(bits_of(c))).astype(np.float16).view(np.uint16)
        ok(fn(p, p, c.data_ptr(), M, N, 0, 1.0, 2.0, stream()))
        assert np.array_equal(bits_of(c), want)


def skinny(d_a, ws, biases, M, K, alpha=1.0):
    import ctypes as C
    outs = [torch.full((M, w.shape[0]), float("nan"), dtype=torch.float16, device="cuda") for w in ws]
    arr = (dev.SkinnyProj * len(ws))()
    for i, (w, b, y) in enumerate(zip(ws, biases, outs)):
        arr[i] = dev.SkinnyProj(w=w.data_ptr(), scales=None, bias=b.data_ptr() if b is not None else None,
                                y=y.data_ptr(), N=w.shape[0])
    st = dev.vv_skinny_linear_dev(d_a.data_ptr(), 0, C.addressof(arr), len(ws), M, K, alpha, stream())
    return st, outs


@pytest.mark.parametrize("M", [9, 29, 64])
@pytest.mark.parametrize("Ns,K,with_bias", [((3584, 512, 512), 3584, True), ((1536, 256), 1536, True),
                                            ((3584,), 18944, False), ((264, 40, 1000), 520, True)])
def test_skinny_linear_equals_gemm_then_bias(M, Ns, K, with_bias):
    """The reference's multi-projection small-M entry point (decoder.c:375, 499):
    one launch, the same bits as vv_gemm_fp16_dev + vv_bias_add_dev per projection."""
    d_a = to_dev(oracle.normal_f16((M, K), 31 + M))
    ws = [to_dev(oracle.normal_f16((n, K), 40 + i, std=K ** -0.5)) for i, n in enumerate(Ns)]
    bs = [to_dev(oracle.normal_f16((n,), 50 + i, std=0.3)) if with_bias and i != 1 else None for i, n in enumerate(Ns)]
    st, outs = skinny(d_a, ws, bs, M, K, alpha=0.5)
    assert st == dev.VV_OK
    for w, b, y in zip(ws, bs, outs):
        n = w.shape[0]
        want = torch.full((M, n), float("nan"), dtype=torch.float16, device="cuda")
        ok(dev.vv_gemm_fp16_dev(d_a.data_ptr(), w.data_ptr(), want.data_ptr(), M, n, K, 0.5, 0.0, stream()))
        if b is not None:
            ok(dev.vv_bias_add_dev(want.data_ptr(), b.data_ptr(), M, n, stream()))
        assert np.array_equal(bits_of(y), bits_of(want))
    # and against the oracle: alpha * A W^T + bias exactly, allowing the two FP16 roundings
    # (product, then sum) and the FP32 accumulation
    prod, mag = exact(bits_of(d_a), bits_of(ws[0]), None, 0.5, 0.0)
    ref = prod + (oracle.widen(bits_of(bs[0])) if bs[0] is not None else 0.0)
    got = oracle.widen(bits_of(outs[0])).astype(np.float64)
    assert scaled_rel_err(got, ref) <= FP16_TOL
    ulp = lambda v: np.spacing(np.abs(v).astype(np.float16)).astype(np.float64)
    bound = 0.5 * ulp(prod) + 0.5 * ulp(ref) + 1e-5 * mag + 2.0 ** -24
    assert np.max(np.abs(got - ref) / bound) <= 1.0


def test_skinny_linear_declines():
    M, K = 29, 512
    d_a = to_dev(oracle.normal_f16((M, K), 1))
    w = to_dev(oracle.normal_f16((256, K), 2))
    wide = to_dev(oracle.normal_f16((12800, K), 3))
    U = dev.VV_ERR_UNSUPPORTED
    assert skinny(d_a, [w], [None], 8, K)[0] == U                       # below 9 rows
    assert skinny(d_a, [w], [None], 65, K)[0] == U
    assert skinny(d_a, [w, wide], [None, None], M, K)[0] == U          # vv_gemm_fp16_dev would tile this one
    assert skinny(d_a, [w] * 3, [None] * 3, M, 500)[0] == U            # K % 8
    import ctypes as C
    arr = (dev.SkinnyProj * 1)(dev.SkinnyProj(w=w.data_ptr(), scales=None, bias=None, y=w.data_ptr(), N=256))
    assert dev.vv_skinny_linear_dev(d_a.data_ptr(), 3, C.addressof(arr), 1, M, K, 1.0, stream()) == U   # no such format
    assert dev.vv_skinny_linear_dev(d_a.data_ptr(), 1, C.addressof(arr), 1, M, K, 1.0, stream()) == dev.VV_ERR_NULL_PTR  # INT8 without scales
    assert dev.vv_skinny_linear_dev(None, 0, C.addressof(arr), 1, M, K, 1.0, stream()) == dev.VV_ERR_NULL_PTR
    torch.cuda.synchronize()


def gemv_multi(d_x, ws, biases, K):
    import ctypes as C
    outs = [torch.full((1, w.shape[0]), float("nan"), dtype=torch.float16, device="cuda") for w in ws]
    arr = (dev.SkinnyProj * len(ws))()
    for i, (w, b, y) in enumerate(zip(ws, biases, outs)):
        arr[i] = dev.SkinnyProj(w=w.data_ptr(), scales=None, bias=b.data_ptr() if b is not None else None,
                                y=y.data_ptr(), N=w.shape[0])
    return dev.vv_gemv_multi_dev(d_x.data_ptr(), C.addressof(arr), len(ws), K, stream()), outs


@pytest.mark.parametrize("Ns,K", [((3584, 512, 512), 3584), ((1536, 256, 256), 1536), ((18944, 18944), 3584),
                                  ((9000,), 520), ((37, 5, 101), 72), ((3584,), 18944), ((37, 5), 8192)])
def test_gemv_multi_equals_gemv_then_bias(Ns, K):
    """One decode row through several projections in one launch == the separate calls, bit for bit."""
    d_x = to_dev(oracle.normal_f16((1, K), 61))
    ws = [to_dev(oracle.normal_f16((n, K), 70 + i, std=K ** -0.5)) for i, n in enumerate(Ns)]
    bs = [to_dev(oracle.normal_f16((n,), 80 + i, std=0.3)) if i != 1 else None for i, n in enumerate(Ns)]
    st, outs = gemv_multi(d_x, ws, bs, K)
    assert st == dev.VV_OK
    for w, b, y in zip(ws, bs, outs):
        n = w.shape[0]
        want = torch.full((1, n), float("nan"), dtype=torch.float16, device="cuda")
        ok(dev.vv_gemm_fp16_dev(d_x.data_ptr(), w.data_ptr(), want.data_ptr(), 1, n, K, 1.0, 0.0, stream()))
        if b is not None:
            ok(dev.vv_bias_add_dev(want.data_ptr(), b.data_ptr(), 1, n, stream()))
        assert np.array_equal(bits_of(y), bits_of(want))
    ref, mag = exact(bits_of(d_x), bits_of(ws[1 if len(ws) > 1 else 0]), None, 1.0, 0.0)     # the bias-free one
    if len(ws) > 1:
        check(bits_of(outs[1]), ref, mag, "gemv multi")


@pytest.mark.parametrize("N,K", [(18944, 3584), (8960, 1536), (100, 64), (9000, 264), (3, 8)])
def test_gemv_swiglu_equals_two_gemvs_and_swiglu(N, K):
    d_x = to_dev(oracle.normal_f16((1, K), 91))
    wg = to_dev(oracle.normal_f16((N, K), 92, std=2.0 * K ** -0.5))
    wu = to_dev(oracle.normal_f16((N, K), 93, std=2.0 * K ** -0.5))
    y = torch.full((1, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_gemv_swiglu_dev(d_x.data_ptr(), wg.data_ptr(), wu.data_ptr(), y.data_ptr(), N, K, stream()))
    g = torch.empty((1, N), dtype=torch.float16, device="cuda")
    u = torch.empty((1, N), dtype=torch.float16, device="cuda")
    ok(dev.vv_gemm_fp16_dev(d_x.data_ptr(), wg.data_ptr(), g.data_ptr(), 1, N, K, 1.0, 0.0, stream()))
    ok(dev.vv_gemm_fp16_dev(d_x.data_ptr(), wu.data_ptr(), u.data_ptr(), 1, N, K, 1.0, 0.0, stream()))
    g_bits, u_bits = bits_of(g), bits_of(u)
    ok(dev.vv_swiglu_dev(g.data_ptr(), u.data_ptr(), g.data_ptr(), N, stream()))
    assert np.array_equal(bits_of(y), bits_of(g))
    # and the oracle's SwiGLU of those FP16 projections
    ref, rne = oracle.swiglu_f16(g_bits, u_bits)
    assert scaled_rel_err(oracle.widen(bits_of(y)), ref) <= FP16_TOL


def test_gemv_multi_declines():
    K = 64
    d_x = to_dev(oracle.normal_f16((1, K), 1))
    narrow, wide = to_dev(oracle.normal_f16((128, K), 2)), to_dev(oracle.normal_f16((16384, K), 3))
    assert gemv_multi(d_x, [narrow, wide], [None, None], K)[0] == dev.VV_ERR_UNSUPPORTED     # two width classes
    assert gemv_multi(d_x, [narrow], [None], 60)[0] == dev.VV_ERR_UNSUPPORTED                 # K % 8
    assert dev.vv_gemv_swiglu_dev(None, narrow.data_ptr(), narrow.data_ptr(), narrow.data_ptr(), 4, K,
                                  stream()) == dev.VV_ERR_NULL_PTR
    torch.cuda.synchronize()
