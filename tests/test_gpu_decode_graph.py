"""A decode step of a small dense decoder (2 layers, 4 query / 2 KV heads of
128) on this library's entry points, captured once as a graph and replayed
token after token, against the same step issued directly on a twin state.

What a replay must get right without re-capture: the position (RoPE angle and
KV-cache row) and the cache length (attention extent, slice boundaries) come
from device memory and advance inside the graph. Every replay is compared with
the eager twin bit for bit (same kernels, so no tolerance), with unrelated
eager work and synchronisations between the replays; the per-op parity against
the CPU oracle is the business of the other GPU tests.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, to_dev

pytestmark = pytest.mark.gpu

H, NQ, NK, HD, I_FF, LAYERS = 512, 4, 2, 128, 1024, 2
QD, KD = NQ * HD, NK * HD
EPS, THETA = 1e-6, 1e4
START = 70            # tokens already in the cache: 2 decode slices up to 128 positions
ROOM = 160


class State:
    """Weights are shared; activations, KV cache and position counters are per state."""

    def __init__(self, weights, seed):
        self.w = weights
        f16 = dict(dtype=torch.float16, device="cuda")
        self.kc = to_dev(oracle.normal_f16((LAYERS, ROOM, NK, HD), seed, std=0.5))
        self.vc = to_dev(oracle.normal_f16((LAYERS, ROOM, NK, HD), seed + 1))
        self.hidden = to_dev(oracle.normal_f16((1, H), seed + 2))
        self.normed, self.proj = torch.empty(1, H, **f16), torch.empty(1, H, **f16)
        self.q, self.attn = torch.empty(1, QD, **f16), torch.empty(1, QD, **f16)
        self.k, self.v = torch.empty(1, KD, **f16), torch.empty(1, KD, **f16)
        self.gate, self.up = torch.empty(1, I_FF, **f16), torch.empty(1, I_FF, **f16)
        self.pos = torch.tensor([START], dtype=torch.int32, device="cuda")
        self.nxt = torch.tensor([START + 1], dtype=torch.int32, device="cuda")
        self.scratch = torch.empty(dev.vv_attn_scratch_bytes(NQ, NK, HD), dtype=torch.uint8, device="cuda")
        self.views = [dev.KvView(k=self.kc[l].data_ptr(), v=self.vc[l].data_ptr(), k_meta=None, v_meta=None,
                                 page_table=None, format=0, n_kv_heads=NK, head_dim=HD) for l in range(LAYERS)]

    def step(self, st, host_cache_len):
        w, P = self.w, (lambda t: t.data_ptr())
        ok = lambda s: s == dev.VV_OK or pytest.fail(f"status {s}")
        gemv = lambda x, wt, y, n, kk: ok(dev.vv_gemm_fp16_dev(P(x), P(wt), P(y), 1, n, kk, 1.0, 0.0, st))
        ok(dev.vv_rmsnorm_dev(P(self.hidden), P(w["n_in"][0]), P(self.normed), 1, H, EPS, st))
        for l in range(LAYERS):
            gemv(self.normed, w["wq"][l], self.q, QD, H)
            gemv(self.normed, w["wk"][l], self.k, KD, H)
            gemv(self.normed, w["wv"][l], self.v, KD, H)
            ok(dev.vv_bias_rope_qk_dev(P(self.q), P(self.k), P(w["bq"][l]), P(w["bk"][l]), 1, NQ, NK, HD, 0,
                                       P(self.pos), THETA, st))
            ok(dev.vv_bias_add_dev(P(self.v), P(w["bv"][l]), 1, KD, st))
            ok(dev.vv_dev_memcpy_d2d_at(P(self.kc[l]), P(self.k), KD * 2, P(self.pos), st))
            ok(dev.vv_dev_memcpy_d2d_at(P(self.vc[l]), P(self.v), KD * 2, P(self.pos), st))
            ok(dev.vv_attn_decode(2, P(self.q), C.addressof(self.views[l]), P(self.attn), NQ, host_cache_len,
                                  P(self.nxt), P(self.scratch), st))
            gemv(self.attn, w["wo"][l], self.proj, H, QD)
            ok(dev.vv_add_rmsnorm_dev(P(self.hidden), P(self.proj), P(w["n_post"][l]), P(self.normed), 1, H, EPS, st))
            gemv(self.normed, w["wg"][l], self.gate, I_FF, H)
            gemv(self.normed, w["wu"][l], self.up, I_FF, H)
            ok(dev.vv_swiglu_dev(P(self.gate), P(self.up), P(self.gate), I_FF, st))
            gemv(self.gate, w["wd"][l], self.proj, H, I_FF)
            ok(dev.vv_add_rmsnorm_dev(P(self.hidden), P(self.proj), P(w["n_in"][l + 1]), P(self.normed), 1, H, EPS, st))
        ok(dev.vv_pos_add_dev(P(self.pos), P(self.pos), 1, st))
        ok(dev.vv_pos_add_dev(P(self.nxt), P(self.nxt), 1, st))


def make_weights():
    n = lambda shape, seed, std, mean=0.0: to_dev(oracle.normal_f16(shape, seed, mean=mean, std=std))
    return {"wq": n((LAYERS, QD, H), 1, H ** -0.5), "wk": n((LAYERS, KD, H), 2, H ** -0.5),
            "wv": n((LAYERS, KD, H), 3, H ** -0.5), "wo": n((LAYERS, H, QD), 4, QD ** -0.5),
            "wg": n((LAYERS, I_FF, H), 5, H ** -0.5), "wu": n((LAYERS, I_FF, H), 6, H ** -0.5),
            "wd": n((LAYERS, H, I_FF), 7, I_FF ** -0.5), "bq": n((LAYERS, QD), 8, 0.1),
            "bk": n((LAYERS, KD), 9, 0.1), "bv": n((LAYERS, KD), 10, 0.1),
            "n_in": n((LAYERS + 1, H), 11, 0.1, 1.0), "n_post": n((LAYERS, H), 12, 0.1, 1.0)}


def test_decode_step_graph_replays_equal_eager_steps():
    weights = make_weights()
    graph_state, eager_state = State(weights, 100), State(weights, 100)
    s = C.c_void_p()
    assert dev.vv_dev_stream_create(C.byref(s)) == dev.VV_OK
    st = s.value
    torch.cuda.synchronize()
    assert dev.vv_attn_decode_shape(2, NQ, NK, START + 1) == dev.vv_attn_decode_shape(2, NQ, NK, START + 8)

    assert dev.vv_dev_graph_begin(st) == dev.VV_OK
    graph_state.step(st, START + 1)                  # the host-side length is baked in; the device int is not
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(st, C.byref(g)) == dev.VV_OK and g.value
    assert int(graph_state.pos.item()) == START      # capture ran nothing

    noise = torch.randn(1 << 20, device="cuda")
    for token in range(6):
        assert dev.vv_dev_graph_launch(g.value, st) == dev.VV_OK
        assert dev.vv_dev_stream_sync(st) == dev.VV_OK
        eager_state.step(st, START + 1 + token)
        assert dev.vv_dev_stream_sync(st) == dev.VV_OK
        noise = (noise * 1.0001).sin_()               # unrelated eager work between replays
        torch.cuda.synchronize()
        assert int(graph_state.pos.item()) == START + 1 + token == int(eager_state.pos.item())
        assert int(graph_state.nxt.item()) == START + 2 + token
        for name in ("hidden", "normed", "attn", "q", "k", "kc", "vc"):
            a, b = getattr(graph_state, name), getattr(eager_state, name)
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"token {token}: {name} differs"
        assert bool(torch.isfinite(graph_state.hidden).all())
    # the six tokens went to rows START .. START + 5 of every layer's cache and nowhere else
    fresh = State(weights, 100)
    touched = (graph_state.kc.view(torch.int16) != fresh.kc.view(torch.int16)).any(dim=-1).any(dim=-1)   # [layer, row]
    want = torch.zeros_like(touched)
    want[:, START:START + 6] = True
    assert torch.equal(touched, want)
    dev.vv_dev_graph_destroy(g.value)
    dev.vv_dev_stream_destroy(st)
