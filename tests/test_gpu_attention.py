"""GPU parity tests of causal GQA attention over an FP16 KV cache (prefill and
decode forms, contiguous and paged) through the C ABI, against the oracle's
restatement of the reference CPU kernel (one pass, online softmax).

Bars: the stated one for FP16 outputs (scaled error <= 2e-3) and an
elementwise one: an output is a convex combination of V rows whose weights the
device rounds to FP16 (2^-11 relative), so |err| <= 1.5e-3 * max|V| plus half
an FP16 ulp. Q is scaled up so the softmax is sharp: a position or mask off by
one moves the result far beyond either bar.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import FP16_TOL, bits_of, dev, ok, stream, to_dev
from conftest import scaled_rel_err

pytestmark = pytest.mark.gpu
FP16, FA1, FA2, FI = 0, 1, 2, 3


def view_of(d_k, d_v, n_kv, hd, table=None, fmt=FP16):
    """A vv_kv_view_t over two device tensors; it keeps them (raw addresses alone would not)."""
    v = dev.KvView(k=d_k.data_ptr(), v=d_v.data_ptr(), k_meta=None, v_meta=None,
                   page_table=table.data_ptr() if table is not None else None,
                   format=fmt, n_kv_heads=n_kv, head_dim=hd)
    v.keep = (d_k, d_v, table)
    return v


def check(got_bits, ref, vmax, what):
    got = oracle.widen(got_bits).astype(np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    err = scaled_rel_err(got, ref)
    assert err <= FP16_TOL, f"{what}: scaled error {err:.3e}"
    with np.errstate(over="ignore"):
        ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    worst = float(np.max(np.abs(got - ref) / (0.5 * ulp + 1.5e-3 * vmax)))
    assert worst <= 1.0, f"{what}: {worst:.3f}x the elementwise bound"


def make(rows, nq, nkv, hd, kv_len, seed, sharp=4.0):
    q = oracle.normal_f16((rows, nq, hd), seed, std=sharp * hd ** -0.25)
    k = oracle.normal_f16((kv_len, nkv, hd), seed + 1, std=hd ** -0.25 * 2.0)
    v = oracle.normal_f16((kv_len, nkv, hd), seed + 2)
    return q, k, v


def prefill(d_q, view, nq, hd, rows, off, kv_len, causal=True, backend=FA2):
    d_o = torch.full((rows, nq, hd), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_attn_prefill(backend, d_q.data_ptr(), C.addressof(view), d_o.data_ptr(), nq, rows, off,
                           kv_len, causal, None, stream()))
    return bits_of(d_o)


PREFILL = [(48, 2, 1, 128, 0, 48, True), (37, 28, 4, 128, 0, 37, True), (200, 8, 2, 128, 100, 300, True),
           (130, 4, 4, 128, 0, 130, True), (5, 28, 4, 128, 1000, 1005, True), (64, 4, 2, 128, 0, 100, False),
           (1, 2, 1, 128, 63, 64, True), (129, 2, 1, 128, 0, 129, True), (23, 14, 2, 128, 24, 48, True),
           (10, 4, 2, 64, 3, 13, True), (7, 6, 3, 96, 0, 7, True), (4, 2, 2, 256, 20, 24, True)]


@pytest.mark.parametrize("rows,nq,nkv,hd,off,kv_len,causal", PREFILL)
def test_prefill_against_oracle(rows, nq, nkv, hd, off, kv_len, causal):
    q, k, v = make(rows, nq, nkv, hd, kv_len, 7 * rows + nq)
    ref = oracle.attention_prefill_f32(oracle.widen(q), oracle.widen(k), oracle.widen(v), off, kv_len, causal)
    d_q = to_dev(q)
    # the cache is longer than kv_len and holds NaN beyond it: nothing past kv_len may be read into the result
    pad = np.full((8, nkv, hd), 0x7E00, np.uint16)
    d_k, d_v = to_dev(np.concatenate([k, pad])), to_dev(np.concatenate([v, pad]))
    vw = view_of(d_k, d_v, nkv, hd)
    vmax = float(np.abs(oracle.widen(v)).max())
    got = prefill(d_q, vw, nq, hd, rows, off, kv_len, causal)
    check(got, ref, vmax, "prefill")
    for backend in (FA1, FI):      # every backend name runs the same kernels
        assert np.array_equal(prefill(d_q, vw, nq, hd, rows, off, kv_len, causal, backend), got)


def test_prefill_sees_exactly_the_causal_window():
    """Changing keys and values after a row's position must not change that row."""
    rows, nq, nkv, hd, off = 70, 4, 2, 128, 30
    kv_len = off + rows
    q, k, v = make(rows, nq, nkv, hd, kv_len, 11)
    d_q = to_dev(q)
    base = prefill(d_q, view_of(to_dev(k), to_dev(v), nkv, hd), nq, hd, rows, off, kv_len)
    k2, v2 = k.copy(), v.copy()
    cut = off + 40                                   # positions >= cut change
    k2[cut:] = oracle.normal_f16(k2[cut:].shape, 99, std=3.0)
    v2[cut:] = oracle.normal_f16(v2[cut:].shape, 98, std=3.0)
    moved = prefill(d_q, view_of(to_dev(k2), to_dev(v2), nkv, hd), nq, hd, rows, off, kv_len)
    assert np.array_equal(moved[:40], base[:40])
    assert not np.array_equal(moved[40:], base[40:])


def paged_cache(k, v, nkv, hd, seed):
    """Scatter a contiguous cache into a shuffled page pool through vv_kv_store_dev."""
    kv_len = k.shape[0]
    n_pages = (kv_len + 63) // 64
    pool_pages = n_pages + 3
    perm = np.random.default_rng(seed).permutation(pool_pages)[:n_pages].astype(np.int32)
    table = torch.zeros(n_pages + 2, dtype=torch.int32, device="cuda")
    ok(dev.vv_kv_page_map_dev(table.data_ptr(), 0, n_pages, perm.ctypes.data, stream()))
    torch.cuda.synchronize()
    assert np.array_equal(table.cpu().numpy()[:n_pages], perm)
    pool_k = torch.full((pool_pages * 64, nkv, hd), float("nan"), dtype=torch.float16, device="cuda")
    pool_v = torch.full((pool_pages * 64, nkv, hd), float("nan"), dtype=torch.float16, device="cuda")
    d_k, d_v = to_dev(k), to_dev(v)
    first = min(kv_len, 70)
    ok(dev.vv_kv_store_dev(d_k.data_ptr(), d_v.data_ptr(), pool_k.data_ptr(), pool_v.data_ptr(), None, None,
                           None, False, nkv, hd, 0, None, first, FP16, table.data_ptr(), stream()))
    if kv_len > first:                              # the rest at a device-side position
        d_pos = torch.tensor([first], dtype=torch.int32, device="cuda")
        row = nkv * hd * 2
        ok(dev.vv_kv_store_dev(d_k.data_ptr() + first * row, d_v.data_ptr() + first * row, pool_k.data_ptr(),
                               pool_v.data_ptr(), None, None, None, False, nkv, hd, 0, d_pos.data_ptr(),
                               kv_len - first, FP16, table.data_ptr(), stream()))
    return pool_k, pool_v, table, perm


@pytest.mark.parametrize("nkv,hd,shift", [(4, 128, 0), (3, 20, 0), (2, 64, 1), (1, 8, 0)])
def test_kv_store_fp16_places_rows(nkv, hd, shift):
    """FP16 append at a host and at a device-side position: rows of whole 16-byte chunks, rows that are not
    (3 x 20 halves), and a source that is not 16-byte aligned (one half off) all land where they belong."""
    cap, n1, n2 = 40, 7, 5
    rng = np.random.default_rng(3)
    k = rng.standard_normal((n1 + n2, nkv, hd)).astype(np.float16)
    v = rng.standard_normal((n1 + n2, nkv, hd)).astype(np.float16)
    flat_k = torch.zeros((n1 + n2) * nkv * hd + 8, dtype=torch.float16, device="cuda")
    flat_v = torch.zeros_like(flat_k)
    flat_k[shift:shift + k.size] = torch.from_numpy(k.reshape(-1)).cuda()
    flat_v[shift:shift + v.size] = torch.from_numpy(v.reshape(-1)).cuda()
    ck = torch.full((cap, nkv, hd), float("nan"), dtype=torch.float16, device="cuda")
    cv = torch.full((cap, nkv, hd), float("nan"), dtype=torch.float16, device="cuda")
    row = nkv * hd * 2
    ok(dev.vv_kv_store_dev(flat_k.data_ptr() + 2 * shift, flat_v.data_ptr() + 2 * shift, ck.data_ptr(), cv.data_ptr(),
                           None, None, None, False, nkv, hd, 3, None, n1, FP16, None, stream()))
    d_pos = torch.tensor([3 + n1], dtype=torch.int32, device="cuda")
    ok(dev.vv_kv_store_dev(flat_k.data_ptr() + 2 * shift + n1 * row, flat_v.data_ptr() + 2 * shift + n1 * row,
                           ck.data_ptr(), cv.data_ptr(), None, None, None, False, nkv, hd, 0, d_pos.data_ptr(), n2,
                           FP16, None, stream()))
    torch.cuda.synchronize()
    got_k, got_v = ck.cpu().numpy(), cv.cpu().numpy()
    assert np.array_equal(got_k[3:3 + n1 + n2].view(np.uint16), k.view(np.uint16))
    assert np.array_equal(got_v[3:3 + n1 + n2].view(np.uint16), v.view(np.uint16))
    assert np.isnan(got_k[:3].astype(np.float32)).all() and np.isnan(got_k[3 + n1 + n2:].astype(np.float32)).all()


@pytest.mark.parametrize("rows,nq,nkv,off", [(100, 4, 2, 150), (1, 28, 4, 300)])
def test_paged_cache_matches_contiguous(rows, nq, nkv, off):
    hd, kv_len = 128, off + rows
    q, k, v = make(rows, nq, nkv, hd, kv_len, 21)
    d_q = to_dev(q)
    pool_k, pool_v, table, perm = paged_cache(k, v, nkv, hd, 5)
    got_pool = bits_of(pool_k).reshape(-1, 64, nkv, hd)
    assert np.array_equal(got_pool[perm[1]], k[64:128])         # the store put page 1 where the table says
    flat = view_of(to_dev(k), to_dev(v), nkv, hd)
    paged = view_of(pool_k, pool_v, nkv, hd, table)
    scratch = torch.empty(dev.vv_attn_scratch_bytes(nq, nkv, hd), dtype=torch.uint8, device="cuda")
    if rows > 1:
        assert np.array_equal(prefill(d_q, paged, nq, hd, rows, off, kv_len),
                              prefill(d_q, flat, nq, hd, rows, off, kv_len))
    else:
        outs = []
        for vw in (flat, paged):
            d_o = torch.zeros((1, nq, hd), dtype=torch.float16, device="cuda")
            ok(dev.vv_attn_decode(FA2, d_q.data_ptr(), C.addressof(vw), d_o.data_ptr(), nq, kv_len, None,
                                  scratch.data_ptr(), stream()))
            outs.append(bits_of(d_o))
        assert np.array_equal(outs[0], outs[1])


# groups of 7, 2, 40 (beyond the streaming kernel), 6, 16 and 12 query heads per KV head; head_dim 64: the generic kernel
@pytest.mark.parametrize("nq,nkv,hd", [(28, 4, 128), (2, 1, 128), (40, 1, 128), (12, 2, 128), (4, 2, 64), (32, 2, 128), (24, 2, 128)])
@pytest.mark.parametrize("cache_len", [1, 17, 64, 65, 255, 257, 1000, 5000, 14449, 40000])
def test_decode_against_oracle(nq, nkv, hd, cache_len):
    q, k, v = make(1, nq, nkv, hd, cache_len, cache_len + nq)
    ref = oracle.attention_prefill_f32(oracle.widen(q), oracle.widen(k), oracle.widen(v), cache_len - 1,
                                       cache_len, True)
    d_q = to_dev(q)
    pad = np.full((300, nkv, hd), 0x7E00, np.uint16)
    d_k, d_v = to_dev(np.concatenate([k, pad])), to_dev(np.concatenate([v, pad]))
    vw = view_of(d_k, d_v, nkv, hd)
    scratch = torch.empty(dev.vv_attn_scratch_bytes(nq, nkv, hd), dtype=torch.uint8, device="cuda")
    d_o = torch.full((1, nq, hd), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_attn_decode(FA2, d_q.data_ptr(), C.addressof(vw), d_o.data_ptr(), nq, cache_len, None,
                          scratch.data_ptr(), stream()))
    vmax = float(np.abs(oracle.widen(v)).max())
    got = bits_of(d_o)
    check(got, ref, vmax, "decode")
    # the exact length from device memory; the host value is only in the same bucket
    shape = dev.vv_attn_decode_shape(FA2, nq, nkv, cache_len)
    host_len = cache_len
    while host_len + 1 <= cache_len + 200 and dev.vv_attn_decode_shape(FA2, nq, nkv, host_len + 1) == shape:
        host_len += 1
    d_len = torch.tensor([cache_len], dtype=torch.int32, device="cuda")
    d_o2 = torch.full((1, nq, hd), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_attn_decode(FA2, d_q.data_ptr(), C.addressof(vw), d_o2.data_ptr(), nq, host_len, d_len.data_ptr(),
                          scratch.data_ptr(), stream()))
    assert np.array_equal(bits_of(d_o2), got)
    # and the prefill form of the same row agrees to FP16 rounding
    one = prefill(d_q, vw, nq, hd, 1, cache_len - 1, cache_len)
    check(one, ref, vmax, "prefill of one row")


def prefill_with_scratch(d_q, view, nq, hd, rows, off, kv_len, scratch):
    d_o = torch.full((rows, nq, hd), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_attn_prefill(FA2, d_q.data_ptr(), C.addressof(view), d_o.data_ptr(), nq, rows, off, kv_len, True,
                           scratch.data_ptr(), stream()))
    return bits_of(d_o)


# few rows against a long cache: with the caller's scratch the keys are cut into runs (a short chunk on top of a
# filled cache, src/inference/decoder.c:1095-1115). Rows, heads, offset: one row tile at the end of a long cache,
# a ragged one, several tiles whose causal limits differ (the last runs are empty for the first tiles), one row.
SPLIT = [(113, 28, 4, 14336), (37, 4, 2, 5000), (300, 4, 1, 3000), (1, 2, 1, 4000), (128, 8, 2, 1000), (600, 4, 2, 700)]


@pytest.mark.parametrize("rows,nq,nkv,off", SPLIT)
def test_prefill_split_over_the_keys(rows, nq, nkv, off):
    hd, kv_len = 128, off + rows
    q, k, v = make(rows, nq, nkv, hd, kv_len, 3 * rows + off)
    ref = oracle.attention_prefill_f32(oracle.widen(q), oracle.widen(k), oracle.widen(v), off, kv_len, True)
    d_q = to_dev(q)
    pad = np.full((8, nkv, hd), 0x7E00, np.uint16)             # NaN past the cache's end
    vw = view_of(to_dev(np.concatenate([k, pad])), to_dev(np.concatenate([v, pad])), nkv, hd)
    vmax = float(np.abs(oracle.widen(v)).max())
    scratch = torch.full((dev.vv_attn_scratch_bytes(nq, nkv, hd) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    got = prefill_with_scratch(d_q, vw, nq, hd, rows, off, kv_len, scratch)
    check(got, ref, vmax, "split prefill")
    assert not np.isnan(scratch[:8].cpu().numpy()).any(), "this shape was meant to take the split path"
    # the one-launch form of the same call agrees to the rounding of the runs' partial sums
    whole = prefill(d_q, vw, nq, hd, rows, off, kv_len)
    d = np.abs(oracle.widen(got).astype(np.float64) - oracle.widen(whole).astype(np.float64))
    assert d.max() <= 2.0 ** -9 * vmax
    # the same bits again, and from a paged cache
    assert np.array_equal(prefill_with_scratch(d_q, vw, nq, hd, rows, off, kv_len, scratch), got)
    pool_k, pool_v, table, _ = paged_cache(k, v, nkv, hd, 9)
    assert np.array_equal(prefill_with_scratch(d_q, view_of(pool_k, pool_v, nkv, hd, table), nq, hd, rows, off, kv_len,
                                               scratch), got)


def test_prefill_scratch_is_left_alone_when_there_is_nothing_to_split():
    """Enough rows to fill the chip, or too few keys for two runs: one launch, the scratch untouched."""
    for rows, nq, nkv, off in ((2048, 28, 4, 0), (64, 4, 2, 100)):
        hd, kv_len = 128, off + rows
        q, k, v = make(rows, nq, nkv, hd, kv_len, 5)
        d_q, vw = to_dev(q), view_of(to_dev(k), to_dev(v), nkv, hd)
        scratch = torch.full((dev.vv_attn_scratch_bytes(nq, nkv, hd) // 4,), float("nan"), dtype=torch.float32, device="cuda")
        got = prefill_with_scratch(d_q, vw, nq, hd, rows, off, kv_len, scratch)
        assert np.array_equal(got, prefill(d_q, vw, nq, hd, rows, off, kv_len))
        assert bool(torch.isnan(scratch).all())


def structured(kind, rows, nq, nkv, hd, kv_len, seed):
    """Scores with a shape along the keys instead of noise alone: the tile kernels form a tile's probabilities on the
    softmax reference as it stands and settle it only where a lane's sum passes 2^15 (attention.hip, RowState), so
    these are the inputs on which that happens in tile after tile, never again after the first, or once, mid-way.
    q is about one in every channel, so a key's score is about the sum of its channels."""
    rng = np.random.default_rng(seed)
    q = (1.0 + 0.05 * rng.standard_normal((rows, nq, hd))).astype(np.float16)
    noise = 0.02 * rng.standard_normal((kv_len, nkv, hd))
    t = np.arange(kv_len, dtype=np.float64)[:, None, None]
    if kind == "rising":          # 5.1 a key raw = 0.65 in base-2 exponents: 42 a tile of 64 keys
        k = 0.04 * t + noise
    elif kind == "falling":       # the first tile holds the maximum; later probabilities fall to nothing
        k = 0.04 * (kv_len - 1 - t) + noise
    else:                         # "spike": noise, one key 49 base-2 exponents above it in the sixth tile
        k = 3.0 * noise
        k[333] = 3.0
    v = rng.standard_normal((kv_len, nkv, hd))
    return bits_of_np(q), bits_of_np(k.astype(np.float16)), bits_of_np(v.astype(np.float16))


def bits_of_np(a):
    return np.ascontiguousarray(a).view(np.uint16)


@pytest.mark.parametrize("kind", ["rising", "falling", "spike"])
@pytest.mark.parametrize("causal", [True, False])
def test_prefill_where_the_softmax_reference_moves(kind, causal):
    rows, nq, nkv, hd, kv_len = 200, 4, 2, 128, 700
    off = kv_len - rows
    q, k, v = structured(kind, rows, nq, nkv, hd, kv_len, 17)
    ref = oracle.attention_prefill_f32(oracle.widen(q), oracle.widen(k), oracle.widen(v), off, kv_len, causal)
    d_q, vw = to_dev(q), view_of(to_dev(k), to_dev(v), nkv, hd)
    vmax = float(np.abs(oracle.widen(v)).max())
    got = prefill(d_q, vw, nq, hd, rows, off, kv_len, causal)
    check(got, ref, vmax, f"{kind} scores")
    # the plain tile kernel: the same state and the same helpers, so the same bits
    import os
    os.environ["VV_ATTN_PREFILL_TILE"] = "1"
    try:
        tile = prefill(d_q, vw, nq, hd, rows, off, kv_len, causal)
    finally:
        os.environ.pop("VV_ATTN_PREFILL_TILE", None)
    assert np.array_equal(tile, got)


@pytest.mark.parametrize("kind", ["rising", "falling", "spike"])
def test_split_prefill_and_decode_where_the_softmax_reference_moves(kind):
    """The runs of a split prefill and the slices of a decode hand on (reference, sum, O) records: their references
    differ by hundreds of base-2 exponents here."""
    rows, nq, nkv, hd, kv_len = 100, 4, 2, 128, 1200
    off = kv_len - rows
    q, k, v = structured(kind, rows, nq, nkv, hd, kv_len, 23)
    ref = oracle.attention_prefill_f32(oracle.widen(q), oracle.widen(k), oracle.widen(v), off, kv_len, True)
    d_q, vw = to_dev(q), view_of(to_dev(k), to_dev(v), nkv, hd)
    vmax = float(np.abs(oracle.widen(v)).max())
    scratch = torch.full((dev.vv_attn_scratch_bytes(nq, nkv, hd) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    got = prefill_with_scratch(d_q, vw, nq, hd, rows, off, kv_len, scratch)
    assert not np.isnan(scratch[:8].cpu().numpy()).any(), "this shape was meant to take the split path"
    check(got, ref, vmax, f"{kind} scores, split prefill")
    # one decode row over the same cache: 4 query heads (the streaming kernel) and 34 on 2 KV heads (the tile
    # kernel's decode form, which shares the prefill's state)
    for heads in (4, 34):
        q1 = np.ascontiguousarray(np.resize(q[-1:], (1, heads, hd)))
        ref1 = oracle.attention_prefill_f32(oracle.widen(q1), oracle.widen(k), oracle.widen(v), kv_len - 1, kv_len, True)
        d_o = torch.full((1, heads, hd), float("nan"), dtype=torch.float16, device="cuda")
        sc = torch.empty(dev.vv_attn_scratch_bytes(heads, nkv, hd), dtype=torch.uint8, device="cuda")
        ok(dev.vv_attn_decode(FA2, to_dev(q1).data_ptr(), C.addressof(vw), d_o.data_ptr(), heads, kv_len, None,
                              sc.data_ptr(), stream()))
        check(bits_of(d_o), ref1, vmax, f"{kind} scores, decode with {heads} heads")


def test_declines_and_edges():
    hd, nkv, nq = 128, 1, 2
    d = torch.zeros((4, nq, hd), dtype=torch.float16, device="cuda")
    vw = view_of(d, d, nkv, hd)
    p = d.data_ptr()
    assert dev.vv_attn_prefill(FA2, None, C.addressof(vw), p, nq, 4, 0, 4, True, None, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_attn_prefill(FA2, p, C.addressof(vw), p, nq, 0, 0, 4, True, None, stream()) == dev.VV_OK
    assert dev.vv_attn_decode(FA2, p, C.addressof(vw), p, nq, 0, None, None, stream()) == dev.VV_OK
    tq = view_of(d, d, nkv, hd, fmt=3)             # a TurboQuant cache without its per-vector scales
    assert dev.vv_attn_prefill(FA2, p, C.addressof(tq), p, nq, 4, 0, 4, True, None, stream()) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_attn_decode(FA2, p, C.addressof(tq), p, nq, 4, None, None, stream()) == dev.VV_ERR_UNSUPPORTED
    odd = view_of(d, d, 3, hd)                     # 2 query heads over 3 KV heads
    assert dev.vv_attn_prefill(FA2, p, C.addressof(odd), p, nq, 4, 0, 4, True, None, stream()) == dev.VV_ERR_UNSUPPORTED
    big = view_of(d, d, nkv, hd)                   # more than one slice needs the scratch
    assert dev.vv_attn_decode(FA2, p, C.addressof(big), p, nq, 4000, None, None, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_kv_store_dev(p, p, p, p, None, None, None, False, nkv, hd, 0, None, 1, 7, None,
                               stream()) == dev.VV_ERR_UNSUPPORTED       # FP32 caches are the CPU path's
    torch.cuda.synchronize()
