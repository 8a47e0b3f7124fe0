"""GPU parity tests of the gated MLP's front half done in one GEMM
(vv_gemm_swiglu_dev: the gate and up projections and the activation of
src/inference/decoder.c:966-977 in one launch).

Bar: BIT FOR BIT against vv_gemm_fp16_dev (gate), vv_gemm_fp16_dev (up) and
vv_swiglu_dev, each of them held to the oracle in test_gpu_gemm.py and
test_gpu_layer_ops.py - for shapes that the separate GEMMs run on their 256x256,
128x128 and 64x64 tiles, ragged rows and columns, the shapes the fused tile does not
serve (which run the three calls through the caller's buffers), and once end to end
against the oracle's own chain.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import bits_of, dev, ok, stream, to_dev

pytestmark = pytest.mark.gpu


def separate(d_a, d_g, d_u, M, N, K):
    gate = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    up = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_gemm_fp16_dev(d_a.data_ptr(), d_g.data_ptr(), gate.data_ptr(), M, N, K, 1.0, 0.0, stream()))
    ok(dev.vv_gemm_fp16_dev(d_a.data_ptr(), d_u.data_ptr(), up.data_ptr(), M, N, K, 1.0, 0.0, stream()))
    ok(dev.vv_swiglu_dev(gate.data_ptr(), up.data_ptr(), out.data_ptr(), M * N, stream()))
    return bits_of(gate), bits_of(up), bits_of(out)


def fused(d_a, d_g, d_u, M, N, K, buffers=True):
    gate = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    up = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    st = dev.vv_gemm_swiglu_dev(d_a.data_ptr(), d_g.data_ptr(), d_u.data_ptr(),
                                gate.data_ptr() if buffers else None, up.data_ptr() if buffers else None,
                                out.data_ptr(), M, N, K, stream())
    return st, bits_of(out), bits_of(gate)


# (M, N, K): the separate GEMMs on 256x256 tiles with a row split, on 128x128 tiles, on 64x64 tiles; ragged rows and
# columns (N % 128, N % 4 and odd N); one slab; many slabs; a 2048-row chunk of a wide layer
SHAPES = [(4100, 2100, 192), (2100, 1100, 64), (300, 520, 128), (65, 37, 64), (130, 1, 128), (257, 130, 64),
          (1000, 258, 3584), (2048, 4736, 256), (70, 4096, 1024)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_fused_equals_the_three_calls(M, N, K):
    d_a = to_dev(oracle.normal_f16((M, K), 11))
    d_g = to_dev(oracle.normal_f16((N, K), 12, std=K ** -0.5))
    d_u = to_dev(oracle.normal_f16((N, K), 13, std=K ** -0.5))
    gate, up, want = separate(d_a, d_g, d_u, M, N, K)
    st, got, gate_buf = fused(d_a, d_g, d_u, M, N, K)
    assert st == dev.VV_OK
    assert np.array_equal(got, want)
    assert np.isnan(oracle.widen(gate_buf)).all(), "the fused tile leaves the buffers alone"
    st, got, _ = fused(d_a, d_g, d_u, M, N, K, buffers=False)       # and does not need them
    assert st == dev.VV_OK and np.array_equal(got, want)


@pytest.mark.parametrize("N,K", [(512, 256), (18944, 3584), (37, 8)])
def test_one_row_runs_the_decode_launch(N, K):
    d_a = to_dev(oracle.normal_f16((1, K), 41))
    d_g = to_dev(oracle.normal_f16((N, K), 42, std=K ** -0.5))
    d_u = to_dev(oracle.normal_f16((N, K), 43, std=K ** -0.5))
    _, _, want = separate(d_a, d_g, d_u, 1, N, K)
    st, got, _ = fused(d_a, d_g, d_u, 1, N, K, buffers=False)
    assert st == dev.VV_OK and np.array_equal(got, want)


@pytest.mark.parametrize("M,N,K", [(64, 300, 128), (9, 100, 64), (2, 512, 256), (200, 96, 72), (300, 64, 8)])
def test_other_shapes_run_the_three_calls(M, N, K):
    """Up to 64 rows, or rows that are not whole 64-half slabs: through the caller's buffers, or declined."""
    d_a = to_dev(oracle.normal_f16((M, K), 21))
    d_g = to_dev(oracle.normal_f16((N, K), 22, std=K ** -0.5))
    d_u = to_dev(oracle.normal_f16((N, K), 23, std=K ** -0.5))
    gate, up, want = separate(d_a, d_g, d_u, M, N, K)
    st, got, gate_buf = fused(d_a, d_g, d_u, M, N, K)
    assert st == dev.VV_OK and np.array_equal(got, want) and np.array_equal(gate_buf, gate)
    st, got, _ = fused(d_a, d_g, d_u, M, N, K, buffers=False)
    assert st == dev.VV_ERR_UNSUPPORTED
    assert np.isnan(oracle.widen(got)).all(), "declined: nothing launched"


@pytest.mark.parametrize("M,N,K", [(24, 18944, 3584), (17, 12800, 64), (64, 13000, 448), (33, 18944, 128), (32, 33000, 64)])
def test_a_streaming_chunk_against_a_wide_n(M, N, K):
    """17 .. 64 rows of whole 64-K lines against an N too wide for the small-M kernel: vv_gemm_fp16_dev streams 128
    columns a workgroup there, and the fused entry point runs that kernel on both matrices at once with SwiGLU in its
    store - the three calls' bits, with or without the gate and up buffers (which it leaves alone)."""
    d_a = to_dev(oracle.normal_f16((M, K), 41))
    d_g = to_dev(oracle.normal_f16((N, K), 42, std=K ** -0.5))
    d_u = to_dev(oracle.normal_f16((N, K), 43, std=K ** -0.5))
    gate, up, want = separate(d_a, d_g, d_u, M, N, K)
    st, got, gate_buf = fused(d_a, d_g, d_u, M, N, K)
    assert st == dev.VV_OK and np.array_equal(got, want)
    assert np.isnan(oracle.widen(gate_buf)).all()
    st, got, _ = fused(d_a, d_g, d_u, M, N, K, buffers=False)
    assert st == dev.VV_OK and np.array_equal(got, want)


def test_against_the_oracle_chain():
    M, N, K = 300, 264, 320
    a, g, u = oracle.normal_f16((M, K), 31), oracle.normal_f16((N, K), 32, std=K ** -0.5), oracle.normal_f16((N, K), 33, std=K ** -0.5)
    st, got, _ = fused(to_dev(a), to_dev(g), to_dev(u), M, N, K)
    assert st == dev.VV_OK
    af = oracle.widen(a).astype(np.float64)
    gate = af @ oracle.widen(g).astype(np.float64).T
    up = af @ oracle.widen(u).astype(np.float64).T
    ref = gate / (1.0 + np.exp(-gate)) * up
    err = np.abs(oracle.widen(got).astype(np.float64) - ref)
    # three FP16 roundings (gate, up, out) of values of this size
    bound = 3.0 * 2.0 ** -11 * (np.abs(ref) + np.abs(up) * 0.3 + np.abs(gate) * np.abs(up)) + 2.0 ** -14
    assert np.all(err <= bound), float((err / bound).max())


def test_arguments():
    p = torch.zeros(16, dtype=torch.float16, device="cuda").data_ptr()
    assert dev.vv_gemm_swiglu_dev(None, p, p, p, p, p, 1, 1, 8, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_gemm_swiglu_dev(p, p, p, p, p, None, 1, 1, 8, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_gemm_swiglu_dev(p, p, p, p, p, p, 0, 4, 8, stream()) == dev.VV_OK
    assert dev.vv_gemm_swiglu_dev(p, p, p, p, p, p, 4, 4, -8, stream()) == dev.VV_ERR_INVALID_ARG
