"""GPU parity tests of the older weight-only linear layers (per-channel INT8,
NF4, INT4 {scale, min}) through the C ABI.

The dequantisers are bit-exact against the oracle's FP16 weights. The one-row
kernels (M <= 8) are held to the FP16 bar against the double-accumulated product
over the oracle's FP32 weights, which is what the reference's own one-row kernels
multiply. From nine rows on a product must equal, bit for bit, dequantising and
then running the dense FP16 GEMM, whichever kernel serves the shape; the small-M
entry point in its INT8 and NF4 formats likewise, bias included.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import FP16_TOL, bits_of, dev, ok, stream, to_dev
from conftest import scaled_rel_err

pytestmark = pytest.mark.gpu

INT8, NF4, AWQ = 1, 2, 3
NAMES = {INT8: "int8", NF4: "nf4", AWQ: "int4"}


def u8(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8)).cuda()


def weight(fmt, N, K, seed, G=128):
    rng = np.random.default_rng(seed)
    w = dict(fmt=fmt, N=N, K=K, G=G)
    if fmt == INT8:
        q = rng.integers(-128, 128, (N, K), dtype=np.int8)
        s = (rng.uniform(0.5, 1.5, N) * K ** -0.5 / 64).astype(np.float32)
        w["w16"], w["w32"] = oracle.int8_dequant(q, s)
        w["d"] = (u8(q), torch.from_numpy(s).cuda(), None)
    elif fmt == NF4:
        p = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        s = oracle.narrow((rng.uniform(0.5, 1.5, N * K // 64) * K ** -0.5 * 2).astype(np.float32))
        w["w16"], w["w32"] = oracle.nf4_dequant(p, s)
        w["d"] = (u8(p), to_dev(s), None)
    else:
        p = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        s = oracle.narrow((rng.uniform(0.2, 1.0, (N, K // G)) * K ** -0.5 / 4).astype(np.float32))
        mn = oracle.narrow(-oracle.widen(s) * rng.integers(0, 16, (N, K // G)))
        w["w16"], w["w32"] = oracle.awq_dequant(p, s, mn, G)
        w["d"] = (u8(p), to_dev(s), to_dev(mn))
    return w


def activations(M, K, seed):
    x = oracle.normal_f16((M, K), seed)
    x.reshape(-1)[:: 257] = oracle.narrow(oracle.widen(x.reshape(-1)[:: 257]) * 24.0)      # a few outliers
    return x


def P(t):
    return t.data_ptr() if t is not None else None


def dequant(w, out):
    q, s, mn = w["d"]
    if w["fmt"] == INT8:
        return dev.vv_dequant_int8_dev(P(q), P(s), P(out), w["N"], w["K"], stream())
    if w["fmt"] == NF4:
        return dev.vv_dequant_nf4_dev(P(q), P(s), P(out), w["N"] * w["K"], 64, stream())
    return dev.vv_dequant_awq_dev(P(q), P(mn), P(s), P(out), w["N"], w["K"], w["G"], stream())


def gemv(w, d_x, d_b, d_y):
    q, s, mn = w["d"]
    if w["fmt"] == INT8:
        return dev.vv_int8_gemv_dev(P(d_x), P(q), P(s), P(d_b), P(d_y), w["N"], w["K"], stream())
    if w["fmt"] == NF4:
        return dev.vv_nf4_gemv_dev(P(d_x), P(q), P(s), P(d_b), P(d_y), w["N"], w["K"], stream())
    return dev.vv_awq_gemv_dev(P(d_x), P(q), P(mn), P(s), P(d_b), P(d_y), w["N"], w["K"], w["G"], stream())


def gemm(w, d_x, d_y, d_tmp, M):
    q, s, mn = w["d"]
    if w["fmt"] == INT8:
        return dev.vv_int8_gemm_dev(P(d_x), P(q), P(s), P(d_y), P(d_tmp), M, w["N"], w["K"], stream())
    if w["fmt"] == NF4:
        return dev.vv_nf4_gemm_dev(P(d_x), P(q), P(s), P(d_y), P(d_tmp), M, w["N"], w["K"], 64, stream())
    return dev.vv_awq_gemm_dev(P(d_x), P(q), P(mn), P(s), P(d_y), P(d_tmp), M, w["N"], w["K"], w["G"], stream())


def check(got_bits, x, weights, bias, what, slack=1e-5):
    """Against the double-accumulated product over `weights` (float array [N][K])."""
    xf = oracle.widen(x).astype(np.float64)
    wf = np.asarray(weights, np.float64)
    ref = xf @ wf.T + (oracle.widen(bias).astype(np.float64) if bias is not None else 0.0)
    mag = np.abs(xf) @ np.abs(wf).T
    got = oracle.widen(got_bits).astype(np.float64)
    err = scaled_rel_err(got, ref)
    assert err <= FP16_TOL, f"{what}: scaled error {err:.3e}"
    with np.errstate(over="ignore"):
        ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    worst = float(np.max(np.abs(got - ref) / (0.5 * ulp + slack * mag + 2.0 ** -25)))
    assert worst <= 1.0, f"{what}: {worst:.3f}x the elementwise bound"


@pytest.mark.parametrize("fmt", [INT8, NF4, AWQ])
@pytest.mark.parametrize("N,K,G", [(8, 64, 32), (77, 256, 64), (512, 3584, 128), (136, 1536, 256)])
def test_dequant_bit_exact(fmt, N, K, G):
    w = weight(fmt, N, K, N + G + fmt, G)
    d_out = torch.full((N, K), float("nan"), dtype=torch.float16, device="cuda")
    ok(dequant(w, d_out))
    assert np.array_equal(bits_of(d_out), w["w16"])


# The one-row kernels multiply the FP32 weight (INT8: exactly; the 4-bit formats
# with the code book or the codes in FP16 and the scale on the partial sum), so
# the bound allows the code book's FP16 rounding: 2^-11 of sum |w||x|.
@pytest.mark.parametrize("fmt", [INT8, NF4, AWQ])
@pytest.mark.parametrize("N,K,G,with_bias", [(3584, 3584, 128, True), (512, 3584, 64, False), (3584, 18944, 128, True),
                                             (18944, 3584, 32, False), (1000, 1536, 256, True), (40, 96, 32, True),
                                             (4, 32, 32, False)])
def test_one_row(fmt, N, K, G, with_bias):
    if fmt == NF4 and K % 64:
        K = 128
    w = weight(fmt, N, K, 3 * N + fmt, G)
    x = activations(1, K, 7 + N)
    bias = oracle.normal_f16((N,), 9, std=0.3) if with_bias else None
    d_x, d_b = to_dev(x), to_dev(bias) if with_bias else None
    d_y = torch.full((N,), float("nan"), dtype=torch.float16, device="cuda")
    ok(gemv(w, d_x, d_b, d_y))
    check(bits_of(d_y)[None, :], x, w["w32"], bias, f"{NAMES[fmt]} gemv {N}x{K}", slack=2.0 ** -11 if fmt == NF4 else 1e-5)


@pytest.mark.parametrize("fmt", [INT8, NF4, AWQ])
@pytest.mark.parametrize("M", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("N,K", [(512, 3584), (264, 1024)])
def test_up_to_eight_rows_need_no_scratch(fmt, M, N, K):
    w = weight(fmt, N, K, M + N + fmt)
    x = activations(M, K, 11 + M)
    d_x = to_dev(x)
    d_y = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(gemm(w, d_x, d_y, None, M))
    check(bits_of(d_y), x, w["w32"], None, f"{NAMES[fmt]} M={M}", slack=2.0 ** -11 if fmt == NF4 else 1e-5)


@pytest.mark.parametrize("fmt", [INT8, NF4, AWQ])
@pytest.mark.parametrize("M,N,K", [(9, 512, 3584), (29, 3584, 3584), (64, 520, 256), (29, 18944, 512), (47, 3584, 1536),
                                   (100, 512, 1024), (300, 1000, 1536), (65, 136, 128)])
def test_gemm_equals_dequantise_then_fp16_gemm(fmt, M, N, K):
    w = weight(fmt, N, K, M + N + 2 * fmt)
    x = activations(M, K, 13 + M)
    d_x = to_dev(x)
    d_tmp = torch.full((N, K), float("nan"), dtype=torch.float16, device="cuda")
    d_y = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(gemm(w, d_x, d_y, d_tmp, M))
    got = bits_of(d_y)
    check(got, x, oracle.widen(w["w16"]), None, f"{NAMES[fmt]} gemm {M}x{N}x{K}")
    d_w = to_dev(w["w16"])
    d_r = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_gemm_fp16_dev(P(d_x), P(d_w), P(d_r), M, N, K, 1.0, 0.0, stream()))
    assert np.array_equal(got, bits_of(d_r))
    if M <= 64:
        # where the small-M kernel serves the shape the scratch is never needed
        d_y2 = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        st = gemm(w, d_x, d_y2, None, M)
        assert st in (dev.VV_OK, dev.VV_ERR_NULL_PTR)
        if st == dev.VV_OK:
            assert np.array_equal(bits_of(d_y2), got)
            assert np.isnan(oracle.widen(bits_of(d_tmp))).all()          # and was not touched above either


@pytest.mark.parametrize("fmt", [INT8, NF4])
@pytest.mark.parametrize("M", [9, 16, 17, 29, 33, 48, 64])
def test_small_m_entry_point_equals_dequantise_gemm_bias(fmt, M):
    """q/k/v-shaped launch in a quantised format (decoder.c:375, 499): one launch,
    the bits of dequantise + vv_gemm_fp16_tile_dev + vv_bias_add_dev per projection."""
    K, Ns = 3584, (3584, 512, 520)
    ws = [weight(fmt, n, K, 50 + i + M) for i, n in enumerate(Ns)]
    bs = [oracle.normal_f16((n,), 60 + i, std=0.3) if i != 1 else None for i, n in enumerate(Ns)]
    x = activations(M, K, 70 + M)
    d_x = to_dev(x)
    d_bs = [to_dev(b) if b is not None else None for b in bs]
    outs = [torch.full((M, n), float("nan"), dtype=torch.float16, device="cuda") for n in Ns]
    arr = (dev.SkinnyProj * 3)()
    for i, (w, b, y) in enumerate(zip(ws, d_bs, outs)):
        arr[i] = dev.SkinnyProj(w=P(w["d"][0]), scales=P(w["d"][1]), bias=P(b), y=P(y), N=w["N"])
    ok(dev.vv_skinny_linear_dev(P(d_x), fmt, C.addressof(arr), 3, M, K, 0.5, stream()))
    for w, b, d_b, y in zip(ws, bs, d_bs, outs):
        d_w = to_dev(w["w16"])
        want = torch.full((M, w["N"]), float("nan"), dtype=torch.float16, device="cuda")
        ok(dev.vv_gemm_fp16_tile_dev(P(d_x), P(d_w), P(want), M, w["N"], K, 0.5, 0.0, stream()))
        if b is not None:
            ok(dev.vv_bias_add_dev(P(want), P(d_b), M, w["N"], stream()))
        assert np.array_equal(bits_of(y), bits_of(want))
    check(bits_of(outs[1]), x, 0.5 * oracle.widen(ws[1]["w16"]), None, f"{NAMES[fmt]} small-M M={M}")


def test_declines_and_null_pointers():
    U, NULL = dev.VV_ERR_UNSUPPORTED, dev.VV_ERR_NULL_PTR
    p = torch.zeros(4096, dtype=torch.float16, device="cuda").data_ptr()
    s = stream()
    assert dev.vv_nf4_gemv_dev(p, p, p, None, p, 8, 48, s) == U                       # K % 32
    assert dev.vv_nf4_gemv_dev(None, p, p, None, p, 8, 64, s) == NULL
    assert dev.vv_nf4_gemm_dev(p, p, p, p, None, 100, 8, 64, 64, s) == NULL            # needs the scratch
    assert dev.vv_nf4_gemm_dev(p, p, p, p, p, 100, 8, 64, 32, s) == U                  # block size
    assert dev.vv_dequant_nf4_dev(p, p, p, 0, 64, s) == dev.VV_ERR_INVALID_ARG
    assert dev.vv_dequant_nf4_dev(p, p, p, 68, 64, s) == U
    assert dev.vv_awq_gemv_dev(p, p, p, p, None, p, 8, 64, 48, s) == U                 # group size
    assert dev.vv_awq_gemm_dev(p, p, None, p, p, p, 4, 8, 64, 32, s) == NULL
    assert dev.vv_dequant_awq_dev(p, p, p, p, 8, 60, 32, s) == U
    assert dev.vv_int8_gemv_dev(p, p, p, None, p, 8, 24, s) == U                       # K % 16
    assert dev.vv_int8_gemm_dev(p, p, p, p, None, 200, 8, 64, s) == NULL
    assert dev.vv_dequant_int8_dev(p, None, p, 8, 64, s) == NULL
