"""GPU test of vv_attn_decode_static, the decode attention entry point that
allocates nothing: its partial states live in a file-scope device array of the
library instead of a caller's scratch buffer.

Checked through the C ABI against vv_attn_decode (caller's scratch) bit for
bit, on two calls in a row, the second with a smaller input, so that whatever
the first call left in the shared array would show; then against the oracle.
The test allocates its tensors before the calls under test and none between
them.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import FP16_TOL, bits_of, dev, ok, stream, to_dev
from conftest import scaled_rel_err

pytestmark = pytest.mark.gpu
FA2 = 2


def _case(nq, nkv, hd, cache_len, seed):
    q = oracle.normal_f16((1, nq, hd), seed, std=4.0 * hd ** -0.25)
    k = oracle.normal_f16((cache_len, nkv, hd), seed + 1, std=hd ** -0.25 * 2.0)
    v = oracle.normal_f16((cache_len, nkv, hd), seed + 2)
    d_q, d_k, d_v = to_dev(q), to_dev(k), to_dev(v)
    view = dev.KvView(k=d_k.data_ptr(), v=d_v.data_ptr(), k_meta=None, v_meta=None, page_table=None,
                      format=0, n_kv_heads=nkv, head_dim=hd)
    scratch = torch.empty(dev.vv_attn_scratch_bytes(nq, nkv, hd), dtype=torch.uint8, device="cuda")
    out_ref = torch.full((1, nq, hd), float("nan"), dtype=torch.float16, device="cuda")
    out_new = torch.full((1, nq, hd), float("nan"), dtype=torch.float16, device="cuda")
    return dict(q=q, k=k, v=v, d_q=d_q, d_k=d_k, d_v=d_v, view=view, scratch=scratch, out_ref=out_ref,
                out_new=out_new, nq=nq, nkv=nkv, hd=hd, cache_len=cache_len)


def _run_pair(c):
    ok(dev.vv_attn_decode(FA2, c["d_q"].data_ptr(), C.addressof(c["view"]), c["out_ref"].data_ptr(), c["nq"],
                          c["cache_len"], None, c["scratch"].data_ptr(), stream()))
    ok(dev.vv_attn_decode_static(FA2, c["d_q"].data_ptr(), C.addressof(c["view"]), c["out_new"].data_ptr(),
                                 c["nq"], c["cache_len"], None, stream()))


def _check(c):
    want, got = bits_of(c["out_ref"]), bits_of(c["out_new"])
    assert np.array_equal(got, want), f"cache {c['cache_len']}: static scratch differs from caller's scratch"
    ref = oracle.attention_prefill_f32(oracle.widen(c["q"]), oracle.widen(c["k"]), oracle.widen(c["v"]),
                                       c["cache_len"] - 1, c["cache_len"], True)
    err = scaled_rel_err(oracle.widen(got).astype(np.float64), np.asarray(ref, dtype=np.float64))
    assert err <= FP16_TOL, f"cache {c['cache_len']}: scaled error {err:.3e} against the oracle"


def test_static_scratch_decode_matches_caller_scratch_twice():
    big = _case(28, 4, 128, 14449, 11)        # 256 slices
    small = _case(12, 2, 128, 3000, 23)       # 64 slices, fewer heads: a subset of the array
    # a first call resolves the array's address (and loads the kernels); from then on the device's free memory -
    # which a hipMalloc inside the library would move, unlike torch's own counters - must stay where it is
    _run_pair(small)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    _run_pair(big)
    _run_pair(small)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_allocated() == before
    _check(big)
    _check(small)
    # the large case again after the small one: nothing stale is read
    big["out_new"].fill_(float("nan"))
    ok(dev.vv_attn_decode_static(FA2, big["d_q"].data_ptr(), C.addressof(big["view"]),
                                 big["out_new"].data_ptr(), 28, 14449, None, stream()))
    assert np.array_equal(bits_of(big["out_new"]), bits_of(big["out_ref"]))


def test_static_scratch_device_length_and_other_paths():
    # the exact length from a device int, inside the host length's bucket
    c = _case(28, 4, 128, 5000, 31)
    d_len = torch.tensor([5000], dtype=torch.int32, device="cuda")
    ok(dev.vv_attn_decode(FA2, c["d_q"].data_ptr(), C.addressof(c["view"]), c["out_ref"].data_ptr(), 28, 5000,
                          None, c["scratch"].data_ptr(), stream()))
    host_len = 5000
    shape = dev.vv_attn_decode_shape(FA2, 28, 4, 5000)
    while host_len < 5100 and dev.vv_attn_decode_shape(FA2, 28, 4, host_len + 1) == shape:
        host_len += 1
    pad = torch.full((host_len - 5000 + 64, 4, 128), float("nan"), dtype=torch.float16, device="cuda")
    d_k, d_v = torch.cat([c["d_k"], pad]), torch.cat([c["d_v"], pad])
    view = dev.KvView(k=d_k.data_ptr(), v=d_v.data_ptr(), k_meta=None, v_meta=None, page_table=None,
                      format=0, n_kv_heads=4, head_dim=128)
    ok(dev.vv_attn_decode_static(FA2, c["d_q"].data_ptr(), C.addressof(view), c["out_new"].data_ptr(), 28,
                                 host_len, d_len.data_ptr(), stream()))
    assert np.array_equal(bits_of(c["out_new"]), bits_of(c["out_ref"]))
    # the shortest split (16 slices) and the generic head_dim: same kernels as vv_attn_decode
    for nq, nkv, hd, n in [(28, 4, 128, 700), (4, 2, 64, 3000)]:
        c = _case(nq, nkv, hd, n, n)
        _run_pair(c)
        _check(c)


def test_static_scratch_limits_and_errors():
    hd, nkv = 128, 1
    nq = dev.VV_ATTN_DECODE_STATIC_MAX_Q_HEADS + 1
    d = torch.zeros((4100, nkv, hd), dtype=torch.float16, device="cuda")
    dq = torch.zeros((1, nq, hd), dtype=torch.float16, device="cuda")
    view = dev.KvView(k=d.data_ptr(), v=d.data_ptr(), k_meta=None, v_meta=None, page_table=None, format=0,
                      n_kv_heads=nkv, head_dim=hd)
    p = dq.data_ptr()
    # beyond the array's size on the split path: a clear error, nothing launched
    assert dev.vv_attn_decode_static(FA2, p, C.addressof(view), p, nq, 4000, None, stream()) == dev.VV_ERR_INVALID_ARG
    assert dev.vv_attn_decode_static(FA2, p, C.addressof(view), p, nq, 600, None, stream()) == dev.VV_ERR_INVALID_ARG
    # the same number of heads at head_dim 64 runs the wave-per-head kernel, which keeps no partial states: served
    d64 = torch.zeros((700, nkv, 64), dtype=torch.float16, device="cuda")
    narrow = dev.KvView(k=d64.data_ptr(), v=d64.data_ptr(), k_meta=None, v_meta=None, page_table=None, format=0,
                        n_kv_heads=nkv, head_dim=64)
    assert dev.vv_attn_decode_static(FA2, p, C.addressof(narrow), p, nq, 600, None, stream()) == dev.VV_OK
    # exactly the maximum is served on the split path
    top = dev.VV_ATTN_DECODE_STATIC_MAX_Q_HEADS
    assert dev.vv_attn_decode_static(FA2, p, C.addressof(view), p, top, 4000, None, stream()) == dev.VV_OK
    assert dev.vv_attn_decode_static(FA2, None, C.addressof(view), p, 2, 600, None, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_attn_decode_static(FA2, p, C.addressof(view), p, 2, 0, None, stream()) == dev.VV_OK
    odd = dev.KvView(k=d.data_ptr(), v=d.data_ptr(), k_meta=None, v_meta=None, page_table=None, format=0,
                     n_kv_heads=3, head_dim=hd)
    assert dev.vv_attn_decode_static(FA2, p, C.addressof(odd), p, 2, 600, None, stream()) == dev.VV_ERR_UNSUPPORTED
    torch.cuda.synchronize()
