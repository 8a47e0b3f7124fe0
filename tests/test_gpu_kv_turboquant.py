"""GPU parity tests of the TurboQuant (4 / 3 / 2 / 1.5 bit) KV cache through the C ABI.

Rotation, store (codes and per-vector RMS) and unpack are held to bit equality
with the oracle, which adds in the accelerator's order. Attention over a
TurboQuant cache must equal, bit for bit, attention over an FP16 cache holding
the unpacked (still rotated) vectors; the dequantiser returns to the original
space as the reference's does; and the whole recipe (rotate Q, attend,
un-rotate the output) must track FP16 attention over the original vectors to
the format's accuracy.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import bits_of, dev, ok, stream, to_dev

pytestmark = pytest.mark.gpu

FA2 = 2
FORMATS = [3, 4, 5, 6]            # VV_KV_TQ4, TQ3, TQ2, TQ1_5
MIN_COS = {3: 0.99, 4: 0.96, 5: 0.89, 6: 0.80}        # the reference's own bars (tests/test_kv_quant.c:125-132)
NKV, HD = 4, 128


def u8(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def qwen_like(n, seed):
    """Keys with a few channels carrying a large, nearly constant component, as
    the reference's own test builds them (tests/test_kv_quant.c:69-83)."""
    rng = np.random.default_rng(seed)
    k = rng.uniform(-2, 2, (n, NKV, HD)).astype(np.float32)
    v = rng.uniform(-1.5, 1.5, (n, NKV, HD)).astype(np.float32)
    k[..., 7] = 60.0 + k[..., 7] * 8.0
    k[..., 33] = -40.0 + k[..., 33] * 4.0
    v[..., 64] *= 6.0
    return oracle.narrow(k), oracle.narrow(v)




def same_attention(a_bits, b_bits, what):
    """A packed cache and the FP16 cache of its decoded values hold the same numbers; their decodes run
    different kernels (the FP16 cache streams, the packed ones go through the LDS tile), so the results
    agree to the rounding of the probabilities (FP16, 2^-11 relative) rather than bit for bit."""
    a, b = oracle.widen(a_bits).astype(np.float64), oracle.widen(b_bits).astype(np.float64)
    err = np.abs(a - b).max() / max(np.abs(b).max(), 1e-9)
    assert err <= 1e-3, f"{what}: packed and FP16 decodes differ by {err:.2e} of the largest output"

def test_rotation_bit_exact_and_inverse():
    x = oracle.normal_f16((5, 28, HD), 1, std=2.0)
    d_x = to_dev(x)
    ok(dev.vv_kv_rotate_dev(d_x.data_ptr(), 28, HD, 5, stream()))
    rotated = bits_of(d_x)
    assert np.array_equal(rotated, oracle.kv_rotate(x))
    ok(dev.vv_kv_unrotate_dev(d_x.data_ptr(), 28, HD, 5, stream()))
    assert np.array_equal(bits_of(d_x), oracle.kv_rotate(rotated, inverse=True))
    assert np.max(np.abs(oracle.widen(bits_of(d_x)) - oracle.widen(x))) < 0.02
    assert dev.vv_kv_rotate_dev(d_x.data_ptr(), 28, 64, 5, stream()) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_kv_rotate_dev(None, 28, HD, 5, stream()) == dev.VV_ERR_NULL_PTR


def store(fmt, k, v, room, pos=0, d_pos=None, ref=None, build=False, table=None):
    n = k.shape[0]
    bpv = oracle.kv_bytes_per_vec(fmt)
    d_k, d_v = to_dev(k), to_dev(v)
    ks = torch.full((room, NKV, bpv), 0xAA, dtype=torch.uint8, device="cuda")
    vs = torch.full((room, NKV, bpv), 0xAA, dtype=torch.uint8, device="cuda")
    km = torch.full((room, NKV), -1.0, dtype=torch.float16, device="cuda")
    vm = torch.full((room, NKV), -1.0, dtype=torch.float16, device="cuda")
    d_ref = to_dev(ref) if ref is not None else (torch.zeros((NKV, HD), dtype=torch.float16, device="cuda") if build else None)
    d_p = torch.tensor([d_pos], dtype=torch.int32, device="cuda") if d_pos is not None else None
    d_t = torch.from_numpy(np.asarray(table, np.int32)).cuda() if table is not None else None
    P = lambda t: t.data_ptr() if t is not None else None
    ok(dev.vv_kv_store_dev(P(d_k), P(d_v), P(ks), P(vs), P(km), P(vm), P(d_ref), build, NKV, HD, pos, P(d_p), n, fmt,
                           P(d_t), stream()))
    torch.cuda.synchronize()
    return dict(ks=ks, vs=vs, km=km, vm=vm, ref=d_ref)


@pytest.mark.parametrize("fmt", FORMATS)
def test_store_and_unpack_bit_exact(fmt):
    n, room = 70, 256
    k, v = qwen_like(n, 3)
    st = store(fmt, k, v, room, build=True)
    ref = oracle.kv_build_ref(k)
    assert np.array_equal(bits_of(st["ref"]), ref)
    want_k, want_km = oracle.kv_store_tq(k, ref, fmt)
    want_v, want_vm = oracle.kv_store_tq(v, None, fmt)
    assert np.array_equal(st["ks"].cpu().numpy()[:n], want_k) and np.array_equal(bits_of(st["km"])[:n], want_km)
    assert np.array_equal(st["vs"].cpu().numpy()[:n], want_v) and np.array_equal(bits_of(st["vm"])[:n], want_vm)
    assert (st["ks"].cpu().numpy()[n:] == 0xAA).all() and (bits_of(st["km"])[n:] == bits_of(st["km"])[-1, -1]).all()
    # back to FP16 in the original space, with and without the reference key
    d_out = torch.zeros((n, NKV, HD), dtype=torch.float16, device="cuda")
    ok(dev.vv_kv_dequant_dev(st["ks"].data_ptr(), st["km"].data_ptr(), None, d_out.data_ptr(), NKV, HD, n, fmt, stream()))
    assert np.array_equal(bits_of(d_out), oracle.kv_dequant(want_k, want_km, None, fmt))
    ok(dev.vv_kv_dequant_dev(st["ks"].data_ptr(), st["km"].data_ptr(), st["ref"].data_ptr(), d_out.data_ptr(), NKV, HD, n,
                             fmt, stream()))
    assert np.array_equal(bits_of(d_out), oracle.kv_dequant(want_k, want_km, ref, fmt))
    # device-side position and pages land the same bytes elsewhere
    st2 = store(fmt, k, v, room, pos=0, d_pos=100, ref=ref)
    assert np.array_equal(st2["ks"].cpu().numpy()[100:100 + n], want_k)
    assert np.array_equal(bits_of(st2["vm"])[100:100 + n], want_vm)
    table = [3, 1, 0, 2]
    st3 = store(fmt, k, v, room, pos=60, ref=ref, table=table)
    ks3, km3 = st3["ks"].cpu().numpy(), bits_of(st3["km"])
    for p in range(n):
        t = 60 + p
        row = table[t // 64] * 64 + t % 64
        assert np.array_equal(ks3[row], want_k[p]) and np.array_equal(km3[row], want_km[p])


def view(k, v, km, vm, fmt, table=None):
    vw = dev.KvView(k=k.data_ptr(), v=v.data_ptr(), k_meta=km.data_ptr() if km is not None else None,
                    v_meta=vm.data_ptr() if vm is not None else None,
                    page_table=table.data_ptr() if table is not None else None, format=fmt, n_kv_heads=NKV, head_dim=HD)
    vw.keep = (k, v, km, vm, table)
    return vw


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("cache_len", [1, 64, 257, 3000])
def test_decode_equals_fp16_cache_of_unpacked_vectors_and_tracks_fp16_attention(fmt, cache_len):
    nq = 28
    k, v = qwen_like(cache_len, 5 + cache_len)
    ref = oracle.kv_build_ref(k)
    ks, km = oracle.kv_store_tq(k, ref, fmt)
    vs, vm = oracle.kv_store_tq(v, None, fmt)
    k16, v16 = oracle.kv_unpack(ks, km, fmt), oracle.kv_unpack(vs, vm, fmt)
    q = oracle.normal_f16((1, nq, HD), 7, std=0.6)
    qr = oracle.kv_rotate(q)
    d_q = to_dev(qr)
    scratch = torch.empty(dev.vv_attn_scratch_bytes(nq, NKV, HD), dtype=torch.uint8, device="cuda")
    outs = []
    for vw in (view(u8(ks), u8(vs), to_dev(km), to_dev(vm), fmt), view(to_dev(k16), to_dev(v16), None, None, 0)):
        d_o = torch.full((1, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
        ok(dev.vv_attn_decode(FA2, d_q.data_ptr(), C.addressof(vw), d_o.data_ptr(), nq, cache_len, None,
                              scratch.data_ptr(), stream()))
        outs.append(bits_of(d_o))
    same_attention(outs[0], outs[1], f"TurboQuant decode, cache {cache_len}")
    # the older entry point, then the recipe's last step
    d_ks, d_vs, d_km, d_vm = u8(ks), u8(vs), to_dev(km), to_dev(vm)
    d_o = torch.full((1, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_gqa_attention_decode_q_dev(d_q.data_ptr(), d_ks.data_ptr(), d_vs.data_ptr(), d_km.data_ptr(),
                                         d_vm.data_ptr(), d_o.data_ptr(), nq, NKV, HD, cache_len, None, fmt,
                                         scratch.data_ptr(), stream()))
    assert np.array_equal(bits_of(d_o), outs[0])
    ok(dev.vv_kv_unrotate_dev(d_o.data_ptr(), nq, HD, 1, stream()))
    got = oracle.widen(bits_of(d_o)).astype(np.float64).ravel()
    # FP16 attention over the original vectors
    d_r = torch.full((1, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
    vw = view(to_dev(k), to_dev(v), None, None, 0)
    d_q0 = to_dev(q)
    ok(dev.vv_attn_decode(FA2, d_q0.data_ptr(), C.addressof(vw), d_r.data_ptr(), nq, cache_len, None, scratch.data_ptr(),
                          stream()))
    want = oracle.widen(bits_of(d_r)).astype(np.float64).ravel()
    cos = float(got @ want / (np.linalg.norm(got) * np.linalg.norm(want) + 1e-30))
    assert cos >= MIN_COS[fmt], cos


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("cache_len", [65, 3000])
def test_decode_bit_for_bit_where_both_caches_run_the_tile_kernel(fmt, cache_len):
    """Seventeen query heads per KV head are more than the FP16 cache's streaming decode kernel takes, so the FP16
    cache of the unpacked vectors runs the tile kernel too: the packed decode must then equal it in every bit."""
    nq = 17 * NKV
    k, v = qwen_like(cache_len, 9 + cache_len)
    ks, km = oracle.kv_store_tq(k, oracle.kv_build_ref(k), fmt)
    vs, vm = oracle.kv_store_tq(v, None, fmt)
    k16, v16 = oracle.kv_unpack(ks, km, fmt), oracle.kv_unpack(vs, vm, fmt)
    d_q = to_dev(oracle.kv_rotate(oracle.normal_f16((1, nq, HD), 13, std=0.6)))
    scratch = torch.empty(dev.vv_attn_scratch_bytes(nq, NKV, HD), dtype=torch.uint8, device="cuda")
    outs = []
    for vw in (view(u8(ks), u8(vs), to_dev(km), to_dev(vm), fmt), view(to_dev(k16), to_dev(v16), None, None, 0)):
        d_o = torch.full((1, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
        ok(dev.vv_attn_decode(FA2, d_q.data_ptr(), C.addressof(vw), d_o.data_ptr(), nq, cache_len, None,
                              scratch.data_ptr(), stream()))
        outs.append(bits_of(d_o))
    assert not np.isnan(oracle.widen(outs[0])).any()
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("fmt", FORMATS)
def test_prefill_equals_fp16_cache_of_unpacked_vectors(fmt):
    nq, q_len, q_offset, kv_len = 28, 70, 130, 200
    k, v = qwen_like(kv_len, 11)
    ks, km = oracle.kv_store_tq(k, None, fmt)
    vs, vm = oracle.kv_store_tq(v, None, fmt)
    k16, v16 = oracle.kv_unpack(ks, km, fmt), oracle.kv_unpack(vs, vm, fmt)
    d_q = to_dev(oracle.kv_rotate(oracle.normal_f16((q_len, nq, HD), 12, std=0.6)))
    outs = []
    for vw in (view(u8(ks), u8(vs), to_dev(km), to_dev(vm), fmt), view(to_dev(k16), to_dev(v16), None, None, 0)):
        d_o = torch.full((q_len, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
        ok(dev.vv_attn_prefill(FA2, d_q.data_ptr(), C.addressof(vw), d_o.data_ptr(), nq, q_len, q_offset, kv_len, True,
                               None, stream()))
        outs.append(bits_of(d_o))
    assert np.array_equal(outs[0], outs[1])
    d_ks, d_vs, d_km, d_vm = u8(ks), u8(vs), to_dev(km), to_dev(vm)
    d_o = torch.full((q_len, nq, HD), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_gqa_attention_prefill_q_dev(d_q.data_ptr(), d_ks.data_ptr(), d_vs.data_ptr(), d_km.data_ptr(),
                                          d_vm.data_ptr(), d_o.data_ptr(), nq, NKV, HD, q_len, q_offset, kv_len, True,
                                          fmt, stream()))
    assert np.array_equal(bits_of(d_o), outs[0])
