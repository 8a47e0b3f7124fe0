"""Several host threads, each on its own stream, calling the ops at once.

The reference runs several inference contexts concurrently from different host
threads on their own streams (include/vibevoice/engine.h:19,
device.h:613-621), so ops must be re-entrant and keep no shared mutable state.
The one piece of host state in this backend is RoPE's frequency table, cached
per thread: the threads below deliberately use different (theta, head_dim)."""
import ctypes as C
import threading

import numpy as np
import pytest
import torch

import oracle
from gpu_util import assert_fp16_close, assert_rope_close, dev, to_dev

pytestmark = pytest.mark.gpu


def test_four_threads_four_streams():
    configs = [(1e6, 128, 28), (1e4, 128, 2), (1e4, 64, 3), (5e5, 256, 5)]
    T, H = 64, 3584
    errors = []
    results = {}
    barrier = threading.Barrier(len(configs))

    def work(idx, theta, hd, heads):
        try:
            torch.cuda.set_device(0)
            st = C.c_void_p()
            assert dev.vv_dev_stream_create(C.byref(st)) == 0
            x = oracle.normal_f16((T, heads, hd), 100 + idx)
            h = oracle.normal_f16((T, H), 200 + idx)
            r = oracle.normal_f16((T, H), 300 + idx)
            w = oracle.normal_f16((H,), 400 + idx, mean=1.0, std=0.1)
            d_x, d_h, d_r, d_w = to_dev(x), to_dev(h), to_dev(r), to_dev(w)
            d_n = torch.empty_like(d_h)
            torch.cuda.synchronize()
            barrier.wait()
            for it in range(50):                       # many interleaved launches
                d_x2 = d_x.clone()
                torch.cuda.current_stream().synchronize()
                assert dev.vv_rope_dev(d_x2.data_ptr(), T, heads, hd, 1000 + idx, None, theta,
                                       st.value) == 0
                d_r2 = d_r.clone()
                torch.cuda.current_stream().synchronize()
                assert dev.vv_add_rmsnorm_dev(d_r2.data_ptr(), d_h.data_ptr(), d_w.data_ptr(),
                                              d_n.data_ptr(), T, H, 1e-6, st.value) == 0
                assert dev.vv_dev_stream_sync(st.value) == 0
            results[idx] = (d_x2.cpu().numpy().view(np.uint16), d_r2.cpu().numpy().view(np.uint16),
                            d_n.cpu().numpy().view(np.uint16), x, h, r, w, theta)
            dev.vv_dev_stream_destroy(st.value)
        except Exception as e:                         # noqa: BLE001
            errors.append((idx, repr(e)))

    threads = [threading.Thread(target=work, args=(i, *c)) for i, c in enumerate(configs)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert len(results) == len(configs)
    for idx, (gx, gr, gn, x, h, r, w, theta) in results.items():
        ref, _ = oracle.rope_f16(x, 1000 + idx, theta)
        assert_rope_close(gx, x, ref, f"thread {idx} rope")
        want_r, nref, nrne = oracle.add_rmsnorm_f16(r, h, w, 1e-6)
        assert np.array_equal(gr, want_r), f"thread {idx} residual"
        assert_fp16_close(gn, nref, nrne, f"thread {idx} add+norm")


def test_threads_run_the_matrix_core_kernels_at_once():
    """Four threads, four streams: the large-tile GEMM (its one-time LDS-size
    attribute is set per thread), the small-M form, a one-row GEMV and prefill
    + decode attention with a scratch of their own. Each thread's results must
    equal what the same calls give alone on the default stream."""
    M_BIG, N, K, NQ, NKV, HD, T = 4100, 8192, 256, 4, 2, 128, 300
    a = to_dev(oracle.normal_f16((M_BIG, K), 1))
    w = to_dev(oracle.normal_f16((N, K), 2, std=K ** -0.5))
    q = to_dev(oracle.normal_f16((T, NQ, HD), 3))
    k = to_dev(oracle.normal_f16((T, NKV, HD), 4))
    v = to_dev(oracle.normal_f16((T, NKV, HD), 5))
    view = dev.KvView(k=k.data_ptr(), v=v.data_ptr(), k_meta=None, v_meta=None, page_table=None, format=0,
                      n_kv_heads=NKV, head_dim=HD)

    def run(st):
        f16 = dict(dtype=torch.float16, device="cuda")
        outs = [torch.zeros(M_BIG, N, **f16), torch.zeros(29, N, **f16), torch.zeros(1, N, **f16),
                torch.zeros(T, NQ, HD, **f16), torch.zeros(1, NQ, HD, **f16)]
        scratch = torch.empty(dev.vv_attn_scratch_bytes(NQ, NKV, HD), dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        for m, o in zip((M_BIG, 29, 1), outs[:3]):
            assert dev.vv_gemm_fp16_dev(a.data_ptr(), w.data_ptr(), o.data_ptr(), m, N, K, 1.0, 0.0, st) == 0
        assert dev.vv_attn_prefill(2, q.data_ptr(), C.addressof(view), outs[3].data_ptr(), NQ, T, 0, T, True,
                                   None, st) == 0
        assert dev.vv_attn_decode(2, q.data_ptr() + (T - 1) * NQ * HD * 2, C.addressof(view), outs[4].data_ptr(),
                                  NQ, T, None, scratch.data_ptr(), st) == 0
        assert dev.vv_dev_stream_sync(st) == 0
        return [o.cpu().numpy().view(np.uint16) for o in outs]

    want = run(None)
    errors, results = [], {}
    barrier = threading.Barrier(4)

    def work(idx):
        try:
            torch.cuda.set_device(0)
            st = C.c_void_p()
            assert dev.vv_dev_stream_create(C.byref(st)) == 0
            barrier.wait()
            for _ in range(5):
                results[idx] = run(st.value)
            dev.vv_dev_stream_destroy(st.value)
        except Exception as e:                         # noqa: BLE001
            errors.append((idx, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for idx in range(4):
        for got, ref in zip(results[idx], want):
            assert np.array_equal(got, ref), f"thread {idx}"
