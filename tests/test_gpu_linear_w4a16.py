"""GPU parity tests of the W4A16 linear layers through the C ABI.

The dequantiser is bit-exact against the oracle ((q - z) * s rounded once to
FP16). The products are FP16 GEMMs over exactly those weights, held to the
FP16 GEMM's bars against the oracle's double-accumulated product: scaled
error <= 2e-3 and elementwise |err| <= half an FP16 ulp + 1e-5 * sum|w||x|.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import FP16_TOL, bits_of, dev, ok, stream, to_dev
from conftest import scaled_rel_err

pytestmark = pytest.mark.gpu


def weight(N, K, G, seed, sym=False):
    rng = np.random.default_rng(seed)
    packed = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    zeros = np.full((N, K // G), 8, np.uint8) if sym else rng.integers(0, 16, (N, K // G), dtype=np.uint8)
    scales = (rng.uniform(0.2, 1.0, (N, K // G)) * K ** -0.5 / 4).astype(np.float16).view(np.uint16)
    gpu, sz = oracle.int4g_to_gpu_layout(packed, scales, zeros, G)
    w16 = oracle.int4g_dequant_f16(packed, scales, zeros, G)
    return dict(N=N, K=K, G=G, w16=w16, d_w=torch.from_numpy(gpu).cuda(), d_sz=torch.from_numpy(sz).cuda())


def activations(M, K, seed):
    x = oracle.normal_f16((M, K), seed)
    x.reshape(-1)[:: 257] = oracle.narrow(oracle.widen(x.reshape(-1)[:: 257]) * 24.0)      # a few outliers
    return x


def check(got_bits, x, w, bias, what):
    xf = oracle.widen(x)
    ref = oracle.gemm_f16w(xf, w["w16"], bias).astype(np.float64)
    mag = np.abs(xf).astype(np.float64) @ np.abs(oracle.widen(w["w16"])).astype(np.float64).T
    got = oracle.widen(got_bits).astype(np.float64)
    err = scaled_rel_err(got, ref)
    assert err <= FP16_TOL, f"{what}: scaled error {err:.3e}"
    with np.errstate(over="ignore"):
        ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    worst = float(np.max(np.abs(got - ref) / (0.5 * ulp + 1e-5 * mag + 2.0 ** -25)))
    assert worst <= 1.0, f"{what}: {worst:.3f}x the elementwise bound"


def gemm(x, w, bias=None, scratch=False):
    M = x.shape[0]
    d_x = to_dev(x)
    d_b = to_dev(bias) if bias is not None else None
    d_y = torch.full((M, w["N"]), float("nan"), dtype=torch.float16, device="cuda")
    d_s = torch.empty(w["N"] * w["K"], dtype=torch.float16, device="cuda") if scratch else None
    ok(dev.vv_w4a16_gemm_dev(d_x.data_ptr(), w["d_w"].data_ptr(), w["d_sz"].data_ptr(),
                             d_b.data_ptr() if d_b is not None else None, d_y.data_ptr(),
                             d_s.data_ptr() if scratch else None, d_s.numel() * 2 if scratch else 0, M, w["N"],
                             w["K"], w["G"], stream()))
    return bits_of(d_y)


def gemv(x, w, bias=None):
    d_x = to_dev(x)
    d_b = to_dev(bias) if bias is not None else None
    d_y = torch.full((w["N"],), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_w4a16_gemv_dev(d_x.data_ptr(), w["d_w"].data_ptr(), w["d_sz"].data_ptr(),
                             d_b.data_ptr() if d_b is not None else None, d_y.data_ptr(), w["N"], w["K"], w["G"],
                             stream()))
    return bits_of(d_y)


@pytest.mark.parametrize("N,K,G", [(8, 32, 32), (77, 256, 64), (512, 3584, 128), (136, 1536, 256), (3584, 3584, 128)])
def test_dequant_bit_exact(N, K, G):
    w = weight(N, K, G, N + G)
    d_out = torch.full((N, K), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_w4a16_dequant_dev(w["d_w"].data_ptr(), w["d_sz"].data_ptr(), d_out.data_ptr(), N, K, G, stream()))
    assert np.array_equal(bits_of(d_out), w["w16"])


WEIGHTS = [(3584, 3584, 128, False), (512, 3584, 128, False), (18944, 3584, 128, False), (3584, 18944, 128, False),
           (1536, 8960, 32, True), (256, 1536, 64, True), (100, 96, 32, False), (8200, 512, 256, False),
           (8216, 320, 64, True)]     # 32 weight rows per workgroup, a scale per chunk pair, a ragged last step


@pytest.mark.parametrize("N,K,G,sym", WEIGHTS)
def test_gemv_and_small_m(N, K, G, sym):
    w = weight(N, K, G, N % 97 + G, sym)
    bias = oracle.normal_f16((N,), 5, std=0.5)
    for M in (1, 2, 3, 7, 8):
        x = activations(M, K, 10 + M)
        got = gemm(x, w, bias)
        check(got, x, w, bias, f"gemm M={M} {N}x{K} g{G}")
        if M == 1:
            alone = gemv(x, w, bias)
            assert np.array_equal(alone.reshape(1, N), got), "one row through either entry point"
            check(gemv(x, w).reshape(1, N), x, w, None, "gemv without bias")


@pytest.mark.parametrize("N,K,G,sym", WEIGHTS[:3] + WEIGHTS[4:])
@pytest.mark.parametrize("M", [9, 16, 28, 64, 65, 285])
def test_gemm_tiles(N, K, G, sym, M):
    if N * K > 3e7 and M != 9:
        pytest.skip("the largest weights at one row count only")
    w = weight(N, K, G, N % 89 + G, sym)
    bias = oracle.normal_f16((N,), 6, std=0.5)
    x = activations(M, K, 20 + M)
    check(gemm(x, w, bias), x, w, bias, f"gemm M={M} {N}x{K} g{G}")


@pytest.mark.parametrize("M,N,K,G", [(2048, 3584, 3584, 128), (4100, 8200, 96, 32), (300, 130, 160, 32)])
def test_gemm_large(M, N, K, G):
    """Enough workgroups for the 256 x 256 tile, ragged edges, K off the 64-column slab."""
    w = weight(N, K, G, 31)
    x = activations(M, K, 32)
    check(gemm(x, w), x, w, None, f"gemm M={M} {N}x{K} g{G}")


@pytest.mark.parametrize("with_bias", [False, True])
def test_gemm_through_the_scratch(with_bias):
    """From 1024 rows a scratch that holds the dense weight is used; the bias
    still joins the FP32 sum before the only rounding, so the bars are the same
    and, the K order being the same, so are the bits."""
    M, N, K, G = 1100, 512, 3584, 128
    w = weight(N, K, G, 33)
    bias = oracle.normal_f16((N,), 8, std=0.5) if with_bias else None
    x = activations(M, K, 34)
    through = gemm(x, w, bias, scratch=True)
    check(through, x, w, bias, "dequantise + FP16 GEMM")
    assert np.array_equal(through, gemm(x, w, bias)), "scratch or not, the same bits"


def test_gemm_prefill_shape_sampled_rows():
    M, N, K, G = 14449, 3584, 3584, 128
    w = weight(N, K, G, 41)
    bias = oracle.normal_f16((N,), 7, std=0.5)
    x = activations(M, K, 42)
    got = gemm(x, w, bias, scratch=True)
    rows = np.sort(np.random.default_rng(2).choice(M, 40, replace=False))
    rows[0], rows[-1] = 0, M - 1
    check(got[rows], x[rows], w, bias, "sampled rows at T = 14449")


@pytest.mark.parametrize("Ns,K,G", [((3584, 512, 512), 3584, 128), ((18944, 18944), 3584, 128), ((1536, 256, 250), 1536, 64),
                                    ((40,), 64, 32)])
def test_gemv_multi_equals_single_calls(Ns, K, G):
    x = activations(1, K, 50)
    d_x = to_dev(x)
    ws = [weight(N, K, G, 60 + i) for i, N in enumerate(Ns)]
    biases = [oracle.normal_f16((N,), 70 + i, std=0.5) if i != 1 else None for i, N in enumerate(Ns)]
    projs = (dev.W4A16Proj * len(Ns))()
    keep = []
    for i, (w, b) in enumerate(zip(ws, biases)):
        d_b = to_dev(b) if b is not None else None
        d_y = torch.full((w["N"],), float("nan"), dtype=torch.float16, device="cuda")
        keep.append((d_b, d_y))
        projs[i] = dev.W4A16Proj(w["d_w"].data_ptr(), w["d_sz"].data_ptr(), d_b.data_ptr() if d_b is not None else None,
                                 d_y.data_ptr(), w["N"])
    ok(dev.vv_w4a16_gemv_multi_dev(d_x.data_ptr(), C.addressof(projs), len(Ns), K, G, stream()))
    for w, b, (_, d_y) in zip(ws, biases, keep):
        got = bits_of(d_y).reshape(1, -1)
        check(got, x, w, b, f"multi N={w['N']}")
        # a row's value does not depend on what else the launch computes: same kernel configuration
        # as one GEMV over the combined row count
    if len(Ns) == 1:
        assert np.array_equal(bits_of(keep[0][1]), gemv(x, ws[0], biases[0]))


def test_gather():
    M, K = 5, 3584
    x = oracle.normal_f16((M, K), 3)
    perm = np.random.default_rng(4).permutation(K).astype(np.int32)
    d_x, d_p = to_dev(x), torch.from_numpy(perm).cuda()
    d_o = torch.zeros((M, K), dtype=torch.float16, device="cuda")
    ok(dev.vv_w4a16_gather_dev(d_x.data_ptr(), d_p.data_ptr(), d_o.data_ptr(), M, K, stream()))
    assert np.array_equal(bits_of(d_o), x[:, perm])
    assert dev.vv_w4a16_gather_dev(d_x.data_ptr(), d_p.data_ptr(), d_o.data_ptr(), M, 36, stream()) == dev.VV_ERR_INVALID_ARG
    assert dev.vv_w4a16_gather_dev(None, d_p.data_ptr(), d_o.data_ptr(), M, K, stream()) == dev.VV_ERR_NULL_PTR


def test_argument_checks_launch_nothing():
    w = weight(64, 128, 32, 1)
    d_x = to_dev(activations(4, 128, 2))
    d_y = torch.full((4, 64), 7.0, dtype=torch.float16, device="cuda")
    X, W, S, Y = d_x.data_ptr(), w["d_w"].data_ptr(), w["d_sz"].data_ptr(), d_y.data_ptr()
    g = dev.vv_w4a16_gemm_dev
    assert g(None, W, S, None, Y, None, 0, 4, 64, 128, 32, stream()) == dev.VV_ERR_NULL_PTR
    assert g(X, W, None, None, Y, None, 0, 4, 64, 128, 32, stream()) == dev.VV_ERR_NULL_PTR
    for G in (0, 16, 48, 512):
        assert g(X, W, S, None, Y, None, 0, 4, 64, 128, G, stream()) == dev.VV_ERR_UNSUPPORTED
    assert g(X, W, S, None, Y, None, 0, 4, 64, 48, 32, stream()) == dev.VV_ERR_UNSUPPORTED      # K % 32
    assert g(X, W, S, None, Y, None, 0, 0, 64, 128, 32, stream()) == dev.VV_ERR_UNSUPPORTED
    assert g(X + 2, W, S, None, Y, None, 0, 1, 64, 96, 32, stream()) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_w4a16_gemv_dev(X, W, S, None, None, 64, 128, 32, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_w4a16_gemv_dev(X, W, S, None, Y, 0, 128, 32, stream()) == dev.VV_ERR_UNSUPPORTED
    projs = (dev.W4A16Proj * 1)(dev.W4A16Proj(W, S, None, Y, 64))
    assert dev.vv_w4a16_gemv_multi_dev(X, C.addressof(projs), 4, 128, 32, stream()) == dev.VV_ERR_INVALID_ARG
    assert dev.vv_w4a16_dequant_dev(W, S, None, 64, 128, 32, stream()) == dev.VV_ERR_NULL_PTR
    torch.cuda.synchronize()
    assert (d_y == 7.0).all()
