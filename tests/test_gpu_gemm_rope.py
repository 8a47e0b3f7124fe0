"""GPU parity tests of the rotary projection done in the GEMM's store
(vv_gemm_bias_rope_dev: the q / k leg of src/inference/decoder.c:825-855 in one
launch) and of the cos/sin table it reads (vv_rope_table_dev).

Bars: the table against FP64 cos/sin of the FP32 angle the reference forms
(src/cpu/cpu_kernels.c:1491-1510), a few FP32 ulps; the fused projection BIT FOR
BIT against vv_gemm_fp16_dev followed by vv_bias_rope_qk_dev (each of them held
to the oracle in test_gpu_gemm.py and test_gpu_layer_ops.py), for every tile
shape, ragged row counts, with and without bias, scalar and device-side position;
and once end to end against the oracle's own chain.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import assert_rope_close, bits_of, dev, ok, stream, to_dev

pytestmark = pytest.mark.gpu

HD = 128


def make_table(rows, off, theta=1e6, d_pos=None, head_dim=HD):
    t = torch.full((rows, head_dim // 2, 2), float("nan"), dtype=torch.float32, device="cuda")
    ok(dev.vv_rope_table_dev(t.data_ptr(), rows, head_dim, 0 if d_pos is not None else off,
                             d_pos.data_ptr() if d_pos is not None else None, theta, stream()))
    return t


@pytest.mark.parametrize("rows,off,hd,theta", [(1, 0, 128, 1e6), (300, 14000, 128, 1e6), (17, 32767, 128, 1e6),
                                               (9, 77, 64, 1e4), (5, 1000, 256, 5e5)])
def test_rope_table_values(rows, off, hd, theta):
    t = make_table(rows, off, theta, head_dim=hd)
    torch.cuda.synchronize()
    got = t.cpu().numpy()
    half = hd // 2
    # the FP32 frequency and the FP32 angle of the reference, then exact cos/sin of that angle
    freq = np.float32(theta) ** (np.float32(-2.0) * np.arange(half, dtype=np.float32) / np.float32(hd))
    freq = freq.astype(np.float32)
    pos = (off + np.arange(rows)).astype(np.float32)
    ang = (pos[:, None] * freq[None, :]).astype(np.float32).astype(np.float64)
    # powf on the host may differ from numpy's float32 power in the last bit: allow the angle that slack
    slack = np.abs(ang) * 2.0 ** -22 + 2.0 ** -22
    assert np.all(np.abs(got[..., 0] - np.cos(ang)) <= slack), "cos"
    assert np.all(np.abs(got[..., 1] - np.sin(ang)) <= slack), "sin"
    if off == 0:
        assert np.array_equal(got[0, :, 0], np.ones(half, np.float32)) and not got[0, :, 1].any()


def reference_chain(d_a, d_w, d_bias, M, heads, K, off, d_pos=None):
    """vv_gemm_fp16_dev, then bias + RoPE: the launches the fused entry point replaces."""
    N = heads * HD
    c = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_gemm_fp16_dev(d_a.data_ptr(), d_w.data_ptr(), c.data_ptr(), M, N, K, 1.0, 0.0, stream()))
    plain = bits_of(c).copy()
    ok(dev.vv_bias_rope_qk_dev(c.data_ptr(), None, d_bias.data_ptr() if d_bias is not None else None, None,
                               M, heads, 0, HD, 0 if d_pos is not None else off,
                               d_pos.data_ptr() if d_pos is not None else None, 1e6, stream()))
    return plain, bits_of(c)


def fused(d_a, d_w, d_bias, M, heads, K, table):
    N = heads * HD
    c = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_gemm_bias_rope_dev(d_a.data_ptr(), d_w.data_ptr(), d_bias.data_ptr() if d_bias is not None else None,
                                 c.data_ptr(), M, heads, HD, K, table.data_ptr(), stream()))
    return bits_of(c)


# (rows, heads, K): the 64x128, 128x128 and 256x256 tiles (K % 32 == 0: copies straight into LDS; else
# through registers), ragged edges in both directions, an odd head count, and row counts up to 64, which
# run the two steps one after the other.
SHAPES = [(65, 1, 64), (100, 4, 3584), (130, 3, 200), (257, 28, 512), (2048, 28, 256), (2048, 4, 3584),
          (4100, 64, 72), (4097, 64, 64), (4100, 63, 96), (4100, 63, 192), (4097, 64, 128), (2048, 148, 64), (19000, 14, 64), (2100, 17, 192), (14449, 4, 128), (2048, 4, 3584), (285, 28, 512), (130, 2, 64), (1, 28, 3584), (29, 4, 3584), (64, 28, 512), (16, 2, 40)]


@pytest.mark.parametrize("M,heads,K", SHAPES)
@pytest.mark.parametrize("with_bias", [True, False])
def test_fused_projection_equals_gemm_then_bias_rope(M, heads, K, with_bias):
    N, off = heads * HD, 913
    a = oracle.normal_f16((M, K), 10 + M)
    w = oracle.normal_f16((N, K), 20 + heads, std=K ** -0.5)
    bias = oracle.normal_f16((N,), 30, std=0.5)
    d_a, d_w = to_dev(a), to_dev(w)
    d_bias = to_dev(bias) if with_bias else None
    plain, want = reference_chain(d_a, d_w, d_bias, M, heads, K, off)
    got = fused(d_a, d_w, d_bias, M, heads, K, make_table(M, off))
    assert np.array_equal(got, want), f"{M}x{N}x{K}: fused store differs from GEMM -> bias + RoPE"
    assert not np.array_equal(got, plain)                      # it rotated something
    # the position read on the device gives the same table, hence the same bytes
    d_pos = torch.tensor([off], dtype=torch.int32, device="cuda")
    got_dev = fused(d_a, d_w, d_bias, M, heads, K, make_table(M, off, d_pos=d_pos))
    assert np.array_equal(got_dev, want)


def test_fused_projection_layer_shapes_against_oracle():
    """Qwen2-7B's q and k projections of one 2048-row prefill chunk at position 8192, against the
    oracle's chain on the device's rounded product (the product itself is held to the oracle in
    test_gpu_gemm.py): bias add bit-exact, rotation inside the rope bound."""
    M, K, off = 2048, 3584, 8192
    a = oracle.normal_f16((M, K), 41)
    d_a = to_dev(a)
    table = make_table(M, off)
    for heads, seed in ((28, 42), (4, 43)):
        N = heads * HD
        w = oracle.normal_f16((N, K), seed, std=K ** -0.5)
        bias = oracle.normal_f16((N,), seed + 10, std=0.5)
        d_w, d_bias = to_dev(w), to_dev(bias)
        plain, want = reference_chain(d_a, d_w, d_bias, M, heads, K, off)
        got = fused(d_a, d_w, d_bias, M, heads, K, table)
        assert np.array_equal(got, want)
        biased = oracle.bias_add_f16(plain, bias).reshape(M, heads, HD)
        ref = oracle.rope_f16(biased, off, 1e6)[0]
        assert_rope_close(got.reshape(M, heads, HD), biased, ref, f"fused projection, {heads} heads")


def test_fused_projection_declines_and_edges():
    M, heads, K = 70, 2, 64
    a, w = to_dev(oracle.normal_f16((M, K), 1)), to_dev(oracle.normal_f16((heads * HD, K), 2))
    table = make_table(M, 0)
    c = torch.zeros((M, heads * HD), dtype=torch.float16, device="cuda")
    st = stream()
    assert dev.vv_gemm_bias_rope_dev(None, w.data_ptr(), None, c.data_ptr(), M, heads, HD, K, table.data_ptr(), st) \
        == dev.VV_ERR_NULL_PTR
    assert dev.vv_gemm_bias_rope_dev(a.data_ptr(), w.data_ptr(), None, c.data_ptr(), M, heads, HD, K, None, st) \
        == dev.VV_ERR_NULL_PTR
    assert dev.vv_gemm_bias_rope_dev(a.data_ptr(), w.data_ptr(), None, c.data_ptr(), M, heads, 64, K,
                                     table.data_ptr(), st) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_gemm_bias_rope_dev(a.data_ptr(), w.data_ptr(), None, c.data_ptr() + 2, M, heads, HD, K,
                                     table.data_ptr(), st) == dev.VV_ERR_UNSUPPORTED
    ok(dev.vv_gemm_bias_rope_dev(a.data_ptr(), w.data_ptr(), None, c.data_ptr(), 0, heads, HD, K, table.data_ptr(), st))
    assert not bits_of(c).any()                                # nothing launched, nothing written
    assert dev.vv_rope_table_dev(None, 4, HD, 0, None, 1e6, st) == dev.VV_ERR_NULL_PTR
    assert dev.vv_rope_table_dev(table.data_ptr(), 4, 7, 0, None, 1e6, st) == dev.VV_ERR_UNSUPPORTED
    # K == 0: the product is zero, so C = rope(bias)
    bias = oracle.normal_f16((heads * HD,), 5, std=0.5)
    d_bias = to_dev(bias)
    ok(dev.vv_gemm_bias_rope_dev(a.data_ptr(), w.data_ptr(), d_bias.data_ptr(), c.data_ptr(), M, heads, HD, 0,
                                 table.data_ptr(), st))
    x = to_dev(np.tile(bias, (M, 1)))
    ok(dev.vv_rope_dev(x.data_ptr(), M, heads, HD, 0, None, 1e6, st))
    assert np.array_equal(bits_of(c), bits_of(x))
