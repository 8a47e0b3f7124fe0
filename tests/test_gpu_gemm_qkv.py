"""GPU parity tests of the q / k / v projections of a prefill chunk done in one
launch (vv_gemm_qkv_rope_dev: src/inference/decoder.c:815-867 on the dense FP16
path - three projections with their biases, RoPE on q and k, the KV append).

Bar: BIT FOR BIT against the launches it replaces - vv_gemm_bias_rope_dev for q
and for k, vv_gemm_fp16_dev + vv_bias_add_dev for v, vv_kv_store_dev for the
append (each held to the oracle in test_gpu_gemm.py, test_gpu_gemm_rope.py,
test_gpu_layer_ops.py and test_gpu_attention.py) - for the shapes the one-grid
tile serves (7 query heads per KV head of 128 channels; more than 64 rows;
K % 64 == 0: one and two workgroups per compute unit, ragged row counts), for
the shapes it does not (which run the separate launches), with and without
biases, into plain buffers, into a contiguous and into a paged FP16 cache, at a
host and at a device-side position; and once end to end against the oracle's own
chain at the layer's shape.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import assert_rope_close, bits_of, dev, ok, stream, to_dev
from test_gpu_gemm_rope import make_table

pytestmark = pytest.mark.gpu
HD = 128


def ptr(t):
    return t.data_ptr() if t is not None else None


def nan16(*shape):
    return torch.full(shape, float("nan"), dtype=torch.float16, device="cuda")


def weights(nq, nkv, K, seed, with_bias):
    mk = lambda n, s: to_dev(oracle.normal_f16((n, K), s, std=K ** -0.5))
    ws = (mk(nq * HD, seed), mk(nkv * HD, seed + 1), mk(nkv * HD, seed + 2))
    if not with_bias:
        return ws, (None, None, None)
    bs = tuple(to_dev(oracle.normal_f16((n,), seed + 3 + i, std=0.5)) for i, n in enumerate((nq * HD, nkv * HD, nkv * HD)))
    return ws, bs


def separate(d_x, ws, bs, M, nq, nkv, K, table):
    """The launches of the reference's call sequence, on this library's entry points."""
    q, k, v = nan16(M, nq * HD), nan16(M, nkv * HD), nan16(M, nkv * HD)
    ok(dev.vv_gemm_bias_rope_dev(d_x.data_ptr(), ws[0].data_ptr(), ptr(bs[0]), q.data_ptr(), M, nq, HD, K,
                                 table.data_ptr(), stream()))
    ok(dev.vv_gemm_bias_rope_dev(d_x.data_ptr(), ws[1].data_ptr(), ptr(bs[1]), k.data_ptr(), M, nkv, HD, K,
                                 table.data_ptr(), stream()))
    ok(dev.vv_gemm_fp16_dev(d_x.data_ptr(), ws[2].data_ptr(), v.data_ptr(), M, nkv * HD, K, 1.0, 0.0, stream()))
    if bs[2] is not None:
        ok(dev.vv_bias_add_dev(v.data_ptr(), bs[2].data_ptr(), M, nkv * HD, stream()))
    return q, k, v


def fused(d_x, ws, bs, M, nq, nkv, K, table, buffers=True, cache=None, page_table=None, pos=0, d_pos=None):
    q = nan16(M, nq * HD)
    k, v = (nan16(M, nkv * HD), nan16(M, nkv * HD)) if buffers else (None, None)
    kc, vc = cache if cache is not None else (None, None)
    st = dev.vv_gemm_qkv_rope_dev(d_x.data_ptr(), ws[0].data_ptr(), ws[1].data_ptr(), ws[2].data_ptr(), ptr(bs[0]),
                                  ptr(bs[1]), ptr(bs[2]), q.data_ptr(), ptr(k), ptr(v), M, nq, nkv, HD, K,
                                  table.data_ptr(), ptr(kc), ptr(vc), ptr(page_table), pos, ptr(d_pos), stream())
    return st, q, k, v


# (rows, query heads, KV heads, K): the layer's chunk (512 tiles: two workgroups per compute unit), its ragged
# neighbour, up to 256 tiles (a workgroup per compute unit, slabs asked for four ahead), one slab, many rows,
# 14 + 2 and 7 + 1 heads
SERVED = [(2048, 28, 4, 3584), (2049, 28, 4, 256), (1000, 28, 4, 3584), (65, 28, 4, 64), (200, 28, 4, 192),
          (4100, 28, 4, 128), (14449, 28, 4, 64), (300, 14, 2, 128), (2100, 14, 2, 64), (130, 7, 1, 320),
          (3000, 7, 1, 64)]
# what the one-grid tile does not serve: another head ratio, up to 64 rows, rows that are not whole 64-half slabs
OTHER = [(300, 12, 2, 128), (64, 28, 4, 128), (1, 28, 4, 3584), (200, 28, 4, 72), (100, 4, 4, 64),
         # 2 .. 64 rows (a streaming chunk): the three projections in one launch of the weight-streaming kernel, one
         # rotation of q and k, the append - whole 64-K lines, another K, two rows, another head ratio
         (24, 28, 4, 3584), (2, 14, 2, 64), (33, 28, 4, 72), (50, 7, 1, 128), (17, 12, 2, 192)]


@pytest.mark.parametrize("M,nq,nkv,K", SERVED + OTHER)
@pytest.mark.parametrize("with_bias", [True, False])
def test_one_launch_equals_the_separate_launches(M, nq, nkv, K, with_bias):
    off = 913
    d_x = to_dev(oracle.normal_f16((M, K), 70 + M))
    ws, bs = weights(nq, nkv, K, 80 + nq, with_bias)
    table = make_table(M, off)
    q, k, v = separate(d_x, ws, bs, M, nq, nkv, K, table)
    st, fq, fk, fv = fused(d_x, ws, bs, M, nq, nkv, K, table)
    assert st == dev.VV_OK
    assert np.array_equal(bits_of(fq), bits_of(q)), "q"
    assert np.array_equal(bits_of(fk), bits_of(k)), "k"
    assert np.array_equal(bits_of(fv), bits_of(v)), "v"


@pytest.mark.parametrize("M,nq,nkv,K", [(2048, 28, 4, 256), (333, 28, 4, 64), (700, 14, 2, 128), (300, 12, 2, 128),
                                      (24, 28, 4, 256)])
@pytest.mark.parametrize("paged", [False, True])
def test_rows_land_in_the_cache(M, nq, nkv, K, paged):
    """The k and v rows in an FP16 cache at positions pos .. pos + M - 1 == vv_kv_store_dev of the separate
    launches' rows; the rest of the cache untouched; position from the host or from the device."""
    pos, cap = 150, 150 + M + 70
    d_x = to_dev(oracle.normal_f16((M, K), 5))
    ws, bs = weights(nq, nkv, K, 6, True)
    table = make_table(M, pos)
    q, k, v = separate(d_x, ws, bs, M, nq, nkv, K, table)
    page_table = None
    if paged:
        n_pages = (cap + 63) // 64
        perm = np.random.default_rng(1).permutation(n_pages + 3)[:n_pages].astype(np.int32)
        page_table = torch.from_numpy(perm).cuda()
        cap = (n_pages + 3) * 64
    want_k, want_v = nan16(cap, nkv, HD), nan16(cap, nkv, HD)
    ok(dev.vv_kv_store_dev(k.data_ptr(), v.data_ptr(), want_k.data_ptr(), want_v.data_ptr(), None, None, None, False,
                           nkv, HD, pos, None, M, 0, ptr(page_table), stream()))
    served = nq == 7 * nkv and M > 64           # up to 64 rows: separate launches, which need the k and v buffers
    for d_pos in (None, torch.tensor([pos], dtype=torch.int32, device="cuda")):
        for buffers in (True, False):
            kc, vc = nan16(cap, nkv, HD), nan16(cap, nkv, HD)
            st, fq, fk, fv = fused(d_x, ws, bs, M, nq, nkv, K, table, buffers=buffers, cache=(kc, vc),
                                   page_table=page_table, pos=0 if d_pos is not None else pos, d_pos=d_pos)
            if not served and not buffers:
                assert st == dev.VV_ERR_UNSUPPORTED          # the separate launches need the k and v buffers
                assert np.isnan(oracle.widen(bits_of(kc))).all(), "declined: nothing launched"
                continue
            assert st == dev.VV_OK
            assert np.array_equal(bits_of(fq), bits_of(q))
            assert np.array_equal(bits_of(kc), bits_of(want_k)) and np.array_equal(bits_of(vc), bits_of(want_v))
            if buffers:
                assert np.array_equal(bits_of(fk), bits_of(k)) and np.array_equal(bits_of(fv), bits_of(v))


def test_layer_shape_against_the_oracle_chain():
    """Qwen2-7B's chunk of 2048 rows at position 8192: the device's rounded products (held to the oracle in
    test_gpu_gemm.py / test_gpu_layer_shapes.py) through the oracle's bias add and rotation."""
    M, nq, nkv, K, off = 2048, 28, 4, 3584, 8192
    x = oracle.normal_f16((M, K), 41)
    d_x = to_dev(x)
    ws, bs = weights(nq, nkv, K, 42, True)
    table = make_table(M, off)
    st, fq, fk, fv = fused(d_x, ws, bs, M, nq, nkv, K, table)
    assert st == dev.VV_OK
    for got, w, b, heads, rotates in ((fq, ws[0], bs[0], nq, True), (fk, ws[1], bs[1], nkv, True),
                                      (fv, ws[2], bs[2], nkv, False)):
        plain = nan16(M, heads * HD)
        ok(dev.vv_gemm_fp16_dev(d_x.data_ptr(), w.data_ptr(), plain.data_ptr(), M, heads * HD, K, 1.0, 0.0, stream()))
        biased = oracle.bias_add_f16(bits_of(plain), bits_of(b))
        if not rotates:
            assert np.array_equal(bits_of(got), biased)
            continue
        biased = biased.reshape(M, heads, HD)
        ref = oracle.rope_f16(biased, off, 1e6)[0]
        assert_rope_close(bits_of(got).reshape(M, heads, HD), biased, ref, f"{heads} heads")
    # sampled rows of v against the oracle's product itself
    rows = [0, 127, 128, 1023, 2047]
    ref = oracle.gemm_f16w(oracle.widen(x[rows]), bits_of(ws[2])).astype(np.float64)
    prod = ref.astype(np.float16).astype(np.float64)
    want = (prod + oracle.widen(bits_of(bs[2])).astype(np.float64))
    err = np.abs(oracle.widen(bits_of(fv)[rows]).astype(np.float64) - want)
    assert np.all(err <= 2.0 ** -10 * (np.abs(want) + np.abs(prod)) + 1e-4)


def test_arguments():
    M, nq, nkv, K = 70, 28, 4, 64
    d_x = to_dev(oracle.normal_f16((M, K), 1))
    ws, bs = weights(nq, nkv, K, 2, True)
    table = make_table(M, 0)
    q, k, v = nan16(M, nq * HD), nan16(M, nkv * HD), nan16(M, nkv * HD)
    st = stream()

    def call(x=d_x.data_ptr(), wq=ws[0].data_ptr(), qq=q.data_ptr(), kk=k.data_ptr(), vv=v.data_ptr(), rows=M,
             hd=HD, kdim=K, tab=table.data_ptr(), kc=None, vc=None, pos=0):
        return dev.vv_gemm_qkv_rope_dev(x, wq, ws[1].data_ptr(), ws[2].data_ptr(), None, None, None, qq, kk, vv, rows,
                                        nq, nkv, hd, kdim, tab, kc, vc, None, pos, None, st)

    assert call(x=None) == dev.VV_ERR_NULL_PTR
    assert call(tab=None) == dev.VV_ERR_NULL_PTR
    assert call(kk=None) == dev.VV_ERR_NULL_PTR                     # neither a k buffer nor a cache
    assert call(kc=k.data_ptr()) == dev.VV_ERR_NULL_PTR             # half a cache
    assert call(hd=64) == dev.VV_ERR_UNSUPPORTED
    assert call(qq=q.data_ptr() + 2) == dev.VV_ERR_UNSUPPORTED
    assert call(kdim=-64) == dev.VV_ERR_INVALID_ARG
    assert call(pos=-1) == dev.VV_ERR_INVALID_ARG
    assert call(rows=0) == dev.VV_OK
    torch.cuda.synchronize()
    assert np.isnan(oracle.widen(bits_of(q))).all(), "nothing launched so far"
    assert call() == dev.VV_OK
    assert not np.isnan(oracle.widen(bits_of(q))).any()
