"""GPU parity tests of the dense layer's matrix-core kernels AT THE SHAPES THE
BENCH LINE QUOTES: prefill attention over 14449 keys (the prompt in one launch
and the reference's 2048-row chunk at offset 12401,
src/inference/decoder.c:869-897, :1166-1174), the FP16 GEMM at the four
projection shapes with 2048 and 14449 rows, and the gate+up+SwiGLU GEMM at
18944 x 3584.

The oracle is O(rows * keys) and single-threaded, so it checks SAMPLED rows -
the first and last rows of the launch and both sides of the 128-row tile edges
at the start, in the middle and at the end - to the bars of
test_gpu_attention.py / test_gpu_gemm.py (the FP64 recipe of the reference's
tests/test_attention.c:94-170). Every element of the full-size outputs is then
tied to those rows by equalities that do not depend on the size: one launch ==
the reference's chunked launches, paged == contiguous, the pipelined kernel ==
the plain tile kernel, GEMM == the 128x128 tile GEMM within the FP32 summation
order, the fused GEMMs == their separate calls bit for bit. Inputs are made on
the device (seeded) and only the sampled rows travel to the host.
"""
import ctypes as C
import os

import numpy as np
import pytest
import torch

import oracle
from gpu_util import FP16_TOL, dev, ok, stream
from conftest import scaled_rel_err

pytestmark = pytest.mark.gpu
FP16_FMT, FA2 = 0, 2
NQ, NKV, HD, H, I = 28, 4, 128, 3584, 18944


def randn16(shape, seed, std=1.0):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * std).to(torch.float16)


def host_f32(t):
    torch.cuda.synchronize()
    return t.detach().float().cpu().numpy()


def same_bits(a, b):
    torch.cuda.synchronize()
    return bool(torch.equal(a.view(torch.int16), b.view(torch.int16)))


def sample_rows(rows, tile=128, seed=0):
    """First / last rows and both sides of the tile edges at the start, middle and end, plus a few others."""
    pick = {0, 1, rows - 1, rows - 2}
    n_tiles = (rows + tile - 1) // tile
    for t in {1, 2, n_tiles // 2, n_tiles // 2 + 1, n_tiles - 2, n_tiles - 1}:
        for d in (-1, 0, 1, 63, 64):
            pick.add(t * tile + d)
    rng = np.random.default_rng(seed)
    pick.update(int(r) for r in rng.integers(0, rows, 12))
    return sorted(r for r in pick if 0 <= r < rows)


# ── prefill attention ──

def view_of(d_k, d_v, table=None):
    v = dev.KvView(k=d_k.data_ptr(), v=d_v.data_ptr(), k_meta=None, v_meta=None,
                   page_table=table.data_ptr() if table is not None else None,
                   format=FP16_FMT, n_kv_heads=NKV, head_dim=HD)
    v.keep = (d_k, d_v, table)
    return v


def prefill(d_q, view, rows, off, kv_len, tile_kernel=False):
    d_o = torch.full((rows, NQ, HD), float("nan"), dtype=torch.float16, device="cuda")
    if tile_kernel:
        os.environ["VV_ATTN_PREFILL_TILE"] = "1"
    try:
        ok(dev.vv_attn_prefill(FA2, d_q.data_ptr(), C.addressof(view), d_o.data_ptr(), NQ, rows, off, kv_len, True,
                               None, stream()))
    finally:
        os.environ.pop("VV_ATTN_PREFILL_TILE", None)
    torch.cuda.synchronize()
    return d_o


def attention_inputs(rows, kv_len, seed):
    # Q scaled up so that the softmax is sharp: a position or a mask off by one moves a row far beyond the bars
    q = randn16((rows, NQ, HD), seed, std=4.0 * HD ** -0.25)
    k = randn16((kv_len, NKV, HD), seed + 1, std=2.0 * HD ** -0.25)
    v = randn16((kv_len, NKV, HD), seed + 2)
    return q, k, v


def check_attention_rows(d_o, d_q, k32, v32, off, picked, what):
    got = host_f32(d_o[picked]).astype(np.float64)
    q32 = host_f32(d_q[picked])
    vmax = float(np.abs(v32).max())
    worst = 0.0
    for i, r in enumerate(picked):
        n = off + r + 1
        ref = oracle.attention_prefill_f32(q32[i:i + 1], k32[:n], v32[:n], off + r, n, True)[0].astype(np.float64)
        err = scaled_rel_err(got[i], ref)
        assert err <= FP16_TOL, f"{what} row {r}: scaled error {err:.3e}"
        with np.errstate(over="ignore"):
            ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
        w = float(np.max(np.abs(got[i] - ref) / (0.5 * ulp + 1.5e-3 * vmax)))
        assert w <= 1.0, f"{what} row {r}: {w:.3f}x the elementwise bound"
        worst = max(worst, w)
    return worst


def paged_copy(d_k, d_v, kv_len, seed):
    """The cache scattered into a shuffled page pool through vv_kv_store_dev."""
    n_pages = (kv_len + 63) // 64
    pool_pages = n_pages + 5
    perm = np.random.default_rng(seed).permutation(pool_pages)[:n_pages].astype(np.int32)
    table = torch.from_numpy(np.concatenate([perm, np.zeros(2, np.int32)])).cuda()
    pool_k = torch.full((pool_pages * 64, NKV, HD), float("nan"), dtype=torch.float16, device="cuda")
    pool_v = torch.full((pool_pages * 64, NKV, HD), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_kv_store_dev(d_k.data_ptr(), d_v.data_ptr(), pool_k.data_ptr(), pool_v.data_ptr(), None, None, None,
                           False, NKV, HD, 0, None, kv_len, FP16_FMT, table.data_ptr(), stream()))
    torch.cuda.synchronize()
    return pool_k, pool_v, table


def test_prefill_chunk_at_the_end_of_the_prompt():
    """The reference's last full chunk: 2048 rows at offset 12401 against 14449 keys."""
    rows, off, kv_len = 2048, 12401, 14449
    d_q, d_k, d_v = attention_inputs(rows, kv_len, 500)
    d_o = prefill(d_q, view_of(d_k, d_v), rows, off, kv_len)
    assert not torch.isnan(d_o).any()
    k32, v32 = host_f32(d_k), host_f32(d_v)
    check_attention_rows(d_o, d_q, k32, v32, off, sample_rows(rows, seed=1), "chunk @12401")
    # the plain tile kernel gives the pipelined kernel's bits, every element
    assert same_bits(prefill(d_q, view_of(d_k, d_v), rows, off, kv_len, tile_kernel=True), d_o)
    # and so does a paged cache
    pool_k, pool_v, table = paged_copy(d_k, d_v, kv_len, 3)
    assert same_bits(prefill(d_q, view_of(pool_k, pool_v, table), rows, off, kv_len), d_o)


def test_prefill_whole_prompt_in_one_launch():
    """14449 rows against 14449 keys (113 row tiles x 226 key tiles): sampled rows against the oracle, every
    element against the reference's own launch pattern - 2048-row chunks at growing offsets."""
    rows = kv_len = 14449
    d_q, d_k, d_v = attention_inputs(rows, kv_len, 600)
    vw = view_of(d_k, d_v)
    d_o = prefill(d_q, vw, rows, 0, kv_len)
    assert not torch.isnan(d_o).any()
    k32, v32 = host_f32(d_k), host_f32(d_v)
    check_attention_rows(d_o, d_q, k32, v32, 0, sample_rows(rows, seed=2), "one launch")
    row_bytes = NQ * HD * 2
    for start in range(0, rows, 2048):
        n = min(2048, rows - start)
        d_c = torch.full((n, NQ, HD), float("nan"), dtype=torch.float16, device="cuda")
        ok(dev.vv_attn_prefill(FA2, d_q.data_ptr() + start * row_bytes, C.addressof(vw), d_c.data_ptr(), NQ, n, start,
                               start + n, True, None, stream()))
        assert same_bits(d_c, d_o[start:start + n]), f"chunk at {start}"
    pool_k, pool_v, table = paged_copy(d_k, d_v, kv_len, 4)
    assert same_bits(prefill(d_q, view_of(pool_k, pool_v, table), rows, 0, kv_len), d_o)


def test_prefill_ragged_chunk():
    """2049 rows at offset 63: a one-row last tile, and no row tile starts on a key tile."""
    rows, off = 2049, 63
    kv_len = off + rows
    d_q, d_k, d_v = attention_inputs(rows, kv_len, 700)
    # the cache is longer than kv_len and holds NaN beyond it
    pad = torch.full((70, NKV, HD), float("nan"), dtype=torch.float16, device="cuda")
    d_kp, d_vp = torch.cat([d_k, pad]), torch.cat([d_v, pad])
    d_o = prefill(d_q, view_of(d_kp, d_vp), rows, off, kv_len)
    assert not torch.isnan(d_o).any()
    check_attention_rows(d_o, d_q, host_f32(d_k), host_f32(d_v), off, sample_rows(rows, seed=3), "ragged")
    assert same_bits(prefill(d_q, view_of(d_kp, d_vp), rows, off, kv_len, tile_kernel=True), d_o)
    pool_k, pool_v, table = paged_copy(d_k, d_v, kv_len, 5)
    assert same_bits(prefill(d_q, view_of(pool_k, pool_v, table), rows, off, kv_len), d_o)


# ── the FP16 GEMM at the layer's shapes ──

LAYER_SHAPES = [(H, H), (NKV * HD, H), (I, H), (H, I)]      # (N, K): q/o, k/v, gate/up, down


def gemm(fn, d_a, d_w, M, N, K):
    d_c = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(fn(d_a.data_ptr(), d_w.data_ptr(), d_c.data_ptr(), M, N, K, 1.0, 0.0, stream()))
    torch.cuda.synchronize()
    return d_c


def check_gemm_rows(d_c, d_a, w_bits, picked, what):
    a32 = host_f32(d_a[picked])
    got = host_f32(d_c[picked]).astype(np.float64)
    ref = oracle.gemm_f16w(a32, w_bits).astype(np.float64)
    mag = np.abs(a32).astype(np.float64) @ np.abs(oracle.widen(w_bits)).astype(np.float64).T
    err = scaled_rel_err(got, ref)
    assert err <= FP16_TOL, f"{what}: scaled error {err:.3e}"
    with np.errstate(over="ignore"):
        ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    worst = float(np.max(np.abs(got - ref) / (0.5 * ulp + 1e-5 * mag + 2.0 ** -25)))
    assert worst <= 1.0, f"{what}: {worst:.3f}x the elementwise bound"


@pytest.mark.parametrize("N,K", LAYER_SHAPES)
@pytest.mark.parametrize("M", [2048, 14449])
def test_gemm_at_the_layer_shapes(M, N, K):
    d_a = randn16((M, K), 1000 + M + N)
    d_w = randn16((N, K), 2000 + N + K, std=K ** -0.5)
    d_c = gemm(dev.vv_gemm_fp16_dev, d_a, d_w, M, N, K)
    assert not torch.isnan(d_c).any()
    torch.cuda.synchronize()
    w_bits = d_w.cpu().numpy().view(np.uint16)
    check_gemm_rows(d_c, d_a, w_bits, sample_rows(M, tile=256, seed=M + N), f"gemm {M}x{N}x{K}")
    # every element: the 128x128 tile GEMM (held to the oracle the same way) adds 16 products at a time where this
    # one adds 32 - the same sums, another rounding of the FP32 partials
    d_t = gemm(dev.vv_gemm_fp16_tile_dev, d_a, d_w, M, N, K)
    check_gemm_rows(d_t, d_a, w_bits, sample_rows(M, tile=256, seed=M + N)[:16], f"tile gemm {M}x{N}x{K}")
    for r0 in range(0, M, 4096):                                # in row blocks: the bound's matrix is FP32
        r1 = min(M, r0 + 4096)
        mag = d_a[r0:r1].float().abs() @ d_w.float().abs().T
        diff = (d_c[r0:r1].float() - d_t[r0:r1].float()).abs()
        assert bool((diff <= 2.0 ** -9 * mag + 2.0 ** -14).all()), "tile shapes must agree to FP32 summation order"
    assert same_bits(gemm(dev.vv_gemm_fp16_dev, d_a, d_w, M, N, K), d_c), "the same call must give the same bits"


@pytest.mark.parametrize("M", [2048, 14449])
def test_gemm_swiglu_at_the_layer_shape(M):
    """gate + up + SwiGLU in one GEMM == the three launches, every element, at 18944 x 3584."""
    N, K = I, H
    d_a = randn16((M, K), 3000 + M)
    d_g = randn16((N, K), 3001, std=K ** -0.5)
    d_u = randn16((N, K), 3002, std=K ** -0.5)
    gate = gemm(dev.vv_gemm_fp16_dev, d_a, d_g, M, N, K)
    up = gemm(dev.vv_gemm_fp16_dev, d_a, d_u, M, N, K)
    want = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_swiglu_dev(gate.data_ptr(), up.data_ptr(), want.data_ptr(), M * N, stream()))
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_gemm_swiglu_dev(d_a.data_ptr(), d_g.data_ptr(), d_u.data_ptr(), None, None, got.data_ptr(), M, N, K,
                              stream()))
    assert same_bits(got, want)
    # sampled rows against the oracle's own chain: FP16 gate and up, then the activation
    picked = sample_rows(M, tile=256, seed=M)[:24]
    a32 = host_f32(d_a[picked])
    g = oracle.gemm_f16w(a32, d_g.cpu().numpy().view(np.uint16)).astype(np.float64)
    u = oracle.gemm_f16w(a32, d_u.cpu().numpy().view(np.uint16)).astype(np.float64)
    ref = g / (1.0 + np.exp(-g)) * u
    err = np.abs(host_f32(got[picked]).astype(np.float64) - ref)
    # three FP16 roundings (gate, up, out) of values of this size
    bound = 3.0 * 2.0 ** -11 * (np.abs(ref) + np.abs(u) * 0.3 + np.abs(g) * np.abs(u)) + 2.0 ** -14
    assert np.all(err <= bound), float((err / bound).max())
