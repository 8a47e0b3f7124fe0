"""GPU parity tests of the FP8 (E4M3 / E5M2) KV cache through the C ABI.

Store and unpack are integer work: bit-exact against the oracle's codec, over
every FP16 input. Attention over an FP8 cache must equal, bit for bit,
attention over an FP16 cache that holds the decoded values (every FP8 value is
an FP16 value and the kernels differ only in how a tile reaches the registers).
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import bits_of, dev, ok, stream, to_dev

pytestmark = pytest.mark.gpu

FA2 = 2
E4M3, E5M2 = 1, 2
NKV, HD = 4, 128


def u8(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def store(fmt, k, v, room, pos=0, d_pos=None, ref=None, build=False, table=None, quant_entry=False):
    """k, v: FP16 bits [n, NKV, HD]. Returns (k_store, v_store, ref) as numpy."""
    n = k.shape[0]
    d_k, d_v = to_dev(k), to_dev(v)
    ks = torch.full((room, NKV, HD), 0xAA, dtype=torch.uint8, device="cuda")
    vs = torch.full((room, NKV, HD), 0xAA, dtype=torch.uint8, device="cuda")
    d_ref = to_dev(ref) if ref is not None else (torch.zeros((NKV, HD), dtype=torch.float16, device="cuda") if build else None)
    d_p = torch.tensor([d_pos], dtype=torch.int32, device="cuda") if d_pos is not None else None
    d_t = torch.from_numpy(np.asarray(table, np.int32)).cuda() if table is not None else None
    P = lambda t: t.data_ptr() if t is not None else None
    if quant_entry:
        ok(dev.vv_kv_quant_store_dev(P(d_k), P(d_v), P(ks), P(vs), None, None, P(d_ref), build, NKV, HD, pos, P(d_p), n,
                                     fmt, stream()))
    else:
        ok(dev.vv_kv_store_dev(P(d_k), P(d_v), P(ks), P(vs), None, None, P(d_ref), build, NKV, HD, pos, P(d_p), n, fmt,
                               P(d_t), stream()))
    torch.cuda.synchronize()
    return ks.cpu().numpy(), vs.cpu().numpy(), (bits_of(d_ref) if d_ref is not None else None)


@pytest.mark.parametrize("fmt", [E4M3, E5M2])
def test_store_every_fp16_value(fmt):
    """All 65536 FP16 patterns as keys and (reversed) as values: zeros, subnormals,
    the saturation edge, infinities and NaNs included."""
    allbits = np.arange(65536, dtype=np.uint16).reshape(128, NKV, HD)
    k, v = allbits, allbits[::-1].copy()
    ks, vs, _ = store(fmt, k, v, 128, quant_entry=True)
    assert np.array_equal(ks, oracle.kv_store_fp8(k, None, fmt == E5M2))
    assert np.array_equal(vs, oracle.kv_store_fp8(v, None, fmt == E5M2))


@pytest.mark.parametrize("fmt", [E4M3, E5M2])
def test_store_with_reference_key_positions_and_pages(fmt):
    n, room = 70, 256
    k = oracle.normal_f16((n, NKV, HD), 1, mean=3.0, std=2.0)
    v = oracle.normal_f16((n, NKV, HD), 2, std=1.5)
    # the first chunk builds the reference key; later chunks reuse it
    ks, vs, ref = store(fmt, k, v, room, build=True)
    want_ref = oracle.kv_build_ref(k)
    assert np.array_equal(ref, want_ref)
    assert np.array_equal(ks[:n], oracle.kv_store_fp8(k, want_ref, fmt == E5M2))
    assert np.array_equal(vs[:n], oracle.kv_store_fp8(v, None, fmt == E5M2))
    assert (ks[n:] == 0xAA).all() and (vs[n:] == 0xAA).all()
    # host position, device position
    for kwargs in (dict(pos=100), dict(pos=0, d_pos=100)):
        ks2, _, _ = store(fmt, k, v, room, ref=want_ref, **kwargs)
        assert np.array_equal(ks2[100:100 + n], ks[:n]) and (ks2[:100] == 0xAA).all()
    # paged: positions 60.. cross from page 0 to page 1 of the table
    table = [3, 1, 0, 2]
    ks3, _, _ = store(fmt, k, v, room, pos=60, ref=want_ref, table=table)
    for p in range(n):
        t = 60 + p
        row = table[t // 64] * 64 + t % 64
        assert np.array_equal(ks3[row], ks[p])


@pytest.mark.parametrize("fmt", [E4M3, E5M2])
def test_dequant(fmt):
    codes = np.arange(256, dtype=np.uint8)
    codes = codes[(codes & 0x7F) <= (0x7E if fmt == E4M3 else 0x7B)]           # what a store can hold
    st = np.resize(codes, (16, NKV, HD)).astype(np.uint8)
    d_out = torch.zeros((16, NKV, HD), dtype=torch.float16, device="cuda")
    d_st = u8(st)
    ok(dev.vv_kv_dequant_dev(d_st.data_ptr(), None, None, d_out.data_ptr(), NKV, HD, 16, fmt, stream()))
    want = oracle.fp8_decode(st, fmt == E5M2)
    assert np.array_equal(oracle.widen(bits_of(d_out)), want)          # FP8 values are FP16 values
    ref = oracle.normal_f16((NKV, HD), 3)
    d_ref = to_dev(ref)
    ok(dev.vv_kv_dequant_dev(d_st.data_ptr(), None, d_ref.data_ptr(), d_out.data_ptr(), NKV, HD, 16, fmt, stream()))
    assert np.array_equal(bits_of(d_out), oracle.narrow(want + oracle.widen(ref)[None]))


def fp8_cache(fmt, n, seed):
    k = oracle.normal_f16((n, NKV, HD), seed, std=1.5)
    v = oracle.normal_f16((n, NKV, HD), seed + 1, std=1.5)
    kq, vq = oracle.kv_store_fp8(k, None, fmt == E5M2), oracle.kv_store_fp8(v, None, fmt == E5M2)
    k16 = oracle.narrow(oracle.fp8_decode(kq, fmt == E5M2))
    v16 = oracle.narrow(oracle.fp8_decode(vq, fmt == E5M2))
    return k, v, kq, vq, k16, v16


def view(k, v, fmt, table=None):
    vw = dev.KvView(k=k.data_ptr(), v=v.data_ptr(), k_meta=None, v_meta=None,
                    page_table=table.data_ptr() if table is not None else None, format=fmt, n_kv_heads=NKV, head_dim=HD)
    vw.keep = (k, v, table)
    return vw


@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("q_len,q_offset,kv_len", [(1, 0, 1), (70, 0, 70), (130, 200, 330), (64, 64, 128), (300, 0, 300)])
def test_prefill_equals_fp16_cache_of_decoded_values(fmt, q_len, q_offset, kv_len):
    nq = 28
    k, v, kq, vq, k16, v16 = fp8_cache(fmt, kv_len, 10 + kv_len)
    q = oracle.normal_f16((q_len, nq, HD), 5)
    d_q = to_dev(q)
    outs = []
    for kk, vv_, f in ((u8(kq), u8(vq), fmt), (to_dev(k16), to_dev(v16), 0)):
        d_o = torch.full((q_len, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
        vw = view(kk, vv_, f)
        ok(dev.vv_attn_prefill(FA2, d_q.data_ptr(), C.addressof(vw), d_o.data_ptr(), nq, q_len, q_offset, kv_len, True,
                               None, stream()))
        outs.append(bits_of(d_o))
    assert np.array_equal(outs[0], outs[1])
    # the older entry point
    d_o = torch.full((q_len, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
    d_kq, d_vq = u8(kq), u8(vq)
    ok(dev.vv_gqa_attention_prefill_q_dev(d_q.data_ptr(), d_kq.data_ptr(), d_vq.data_ptr(), None, None,
                                          d_o.data_ptr(), nq, NKV, HD, q_len, q_offset, kv_len, True, fmt, stream()))
    assert np.array_equal(bits_of(d_o), outs[0])
    # and it is attention over the unquantised cache to FP8 precision
    d_r = torch.full((q_len, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
    vw = view(to_dev(k), to_dev(v), 0)
    ok(dev.vv_attn_prefill(FA2, d_q.data_ptr(), C.addressof(vw), d_r.data_ptr(), nq, q_len, q_offset, kv_len, True,
                           None, stream()))
    err = np.abs(oracle.widen(outs[0]) - oracle.widen(bits_of(d_r))).max()
    assert err < (0.5 if fmt == E4M3 else 1.0), err      # half a step of a value near 6: 3 or 2 mantissa bits


def same_attention(a_bits, b_bits, what):
    """A packed cache and the FP16 cache of its decoded values hold the same numbers; their decodes run
    different kernels (the FP16 cache streams, the packed ones go through the LDS tile), so the results
    agree to the rounding of the probabilities (FP16, 2^-11 relative) rather than bit for bit."""
    a, b = oracle.widen(a_bits).astype(np.float64), oracle.widen(b_bits).astype(np.float64)
    err = np.abs(a - b).max() / max(np.abs(b).max(), 1e-9)
    assert err <= 1e-3, f"{what}: packed and FP16 decodes differ by {err:.2e} of the largest output"


@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("cache_len,paged", [(1, False), (64, False), (65, False), (1500, False), (14449, False), (700, True)])
def test_decode_equals_fp16_cache_of_decoded_values(fmt, cache_len, paged):
    nq = 28
    room = (cache_len + 63) // 64 * 64
    k, v, kq, vq, k16, v16 = fp8_cache(fmt, cache_len, 20 + cache_len % 97)
    table = None
    if paged:
        perm = np.random.default_rng(4).permutation(room // 64).astype(np.int32)
        table = torch.from_numpy(perm).cuda()

        def scatter(a):
            out = np.zeros((room,) + a.shape[1:], a.dtype)
            for t in range(cache_len):
                out[perm[t // 64] * 64 + t % 64] = a[t]
            return out
        kq, vq, k16, v16 = scatter(kq), scatter(vq), scatter(k16), scatter(v16)
    q = oracle.normal_f16((1, nq, HD), 6)
    d_q = to_dev(q)
    scratch = torch.empty(dev.vv_attn_scratch_bytes(nq, NKV, HD), dtype=torch.uint8, device="cuda")
    d_len = torch.tensor([cache_len], dtype=torch.int32, device="cuda")
    outs = []
    for kk, vv_, f in ((u8(kq), u8(vq), fmt), (to_dev(k16), to_dev(v16), 0)):
        d_o = torch.full((1, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
        vw = view(kk, vv_, f, table)
        ok(dev.vv_attn_decode(FA2, d_q.data_ptr(), C.addressof(vw), d_o.data_ptr(), nq, cache_len, d_len.data_ptr(),
                              scratch.data_ptr(), stream()))
        outs.append(bits_of(d_o))
    same_attention(outs[0], outs[1], f"fp8 decode, cache {cache_len}")
    if not paged:
        d_o = torch.full((1, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
        d_kq, d_vq = u8(kq), u8(vq)
        ok(dev.vv_gqa_attention_decode_q_dev(d_q.data_ptr(), d_kq.data_ptr(), d_vq.data_ptr(), None, None,
                                             d_o.data_ptr(), nq, NKV, HD, cache_len, None, fmt, scratch.data_ptr(),
                                             stream()))
        assert np.array_equal(bits_of(d_o), outs[0])


@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("cache_len", [65, 1500, 14449])
def test_decode_bit_for_bit_where_both_caches_run_the_tile_kernel(fmt, cache_len):
    """Seventeen query heads per KV head are more than the FP16 cache's streaming decode kernel takes, so the FP16
    cache of the decoded values runs the tile kernel too: the packed decode must then equal it in every bit -
    one wrong code on a small channel would show."""
    nq = 17 * NKV
    k, v, kq, vq, k16, v16 = fp8_cache(fmt, cache_len, 40 + cache_len % 89)
    d_q = to_dev(oracle.normal_f16((1, nq, HD), 8))
    scratch = torch.empty(dev.vv_attn_scratch_bytes(nq, NKV, HD), dtype=torch.uint8, device="cuda")
    outs = []
    for kk, vv_, f in ((u8(kq), u8(vq), fmt), (to_dev(k16), to_dev(v16), 0)):
        d_o = torch.full((1, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
        vw = view(kk, vv_, f)
        ok(dev.vv_attn_decode(FA2, d_q.data_ptr(), C.addressof(vw), d_o.data_ptr(), nq, cache_len, None,
                              scratch.data_ptr(), stream()))
        outs.append(bits_of(d_o))
    assert not np.isnan(oracle.widen(outs[0])).any()
    assert np.array_equal(outs[0], outs[1])


def test_formats_and_shapes_not_served():
    P = torch.zeros(4096, dtype=torch.float16, device="cuda").data_ptr()
    for fmt in (7, 9):                # FP32 (the CPU path's), no such format
        assert dev.vv_kv_quant_store_dev(P, P, P, P, P, P, None, False, NKV, HD, 0, None, 1, fmt, stream()) == dev.VV_ERR_UNSUPPORTED
        assert dev.vv_kv_dequant_dev(P, P, None, P, NKV, HD, 1, fmt, stream()) == dev.VV_ERR_UNSUPPORTED
        assert dev.vv_gqa_attention_decode_q_dev(P, P, P, P, P, P, 28, NKV, HD, 10, None, fmt, P, stream()) == dev.VV_ERR_UNSUPPORTED
        assert dev.vv_gqa_attention_prefill_q_dev(P, P, P, P, P, P, 28, NKV, HD, 4, 0, 4, True, fmt, stream()) == dev.VV_ERR_UNSUPPORTED
        assert dev.vv_attn_resolve(FA2, fmt, False, 28, NKV, HD) == 1
    assert dev.vv_kv_quant_store_dev(P, P, P, P, None, None, None, False, NKV, HD, 0, None, 1, 0, stream()) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_kv_quant_store_dev(P, P, P, P, None, None, None, False, NKV, 64, 0, None, 1, E4M3, stream()) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_kv_quant_store_dev(None, P, P, P, None, None, None, False, NKV, HD, 0, None, 1, E4M3, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_attn_resolve(FA2, E4M3, True, 28, NKV, HD) == FA2 and dev.vv_attn_resolve(FA2, E5M2, False, 28, NKV, 64) == 1
    assert dev.vv_gqa_attention_decode_q_dev(P, P, P, None, None, P, 28, NKV, HD, 0, None, E4M3, P, stream()) == dev.VV_OK
    # TurboQuant needs the per-vector scales
    assert dev.vv_gqa_attention_decode_q_dev(P, P, P, None, None, P, 28, NKV, HD, 10, None, 3, P, stream()) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_kv_dequant_dev(P, None, None, P, NKV, HD, 1, 3, stream()) == dev.VV_ERR_NULL_PTR
