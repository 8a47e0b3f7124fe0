"""The layer ops composed in the decoder's order, on a tiny random dense model.

Mirrors what the reference's tests/test_prefill_append.c checks for a backend
(GPU ≈ CPU on a model of HS=256, 2 heads x 128, 1 KV head, INTER=512, 2 layers,
theta 1e4; :30,70,269,282), restricted to what this library owns: every
transformer-layer op below is a call into libvibevoice_hip.so through the C
ABI, in the order and with the buffer aliasing of decoder_layer_impl
(src/inference/decoder.c:804-990: norm -> q/k/v -> RoPE -> attention -> o_proj
-> residual -> norm -> gate/up -> SwiGLU in place -> down -> residual). The
projections and the attention are NOT this library's: torch stands in for them
on the device and numpy on the host, identically in every variant.

Checks: (1) the fused entry points give the same bits as the reference-API
sequence over the whole chain; (2) the device chain agrees with the CPU chain
(oracle ops, FP32 activations) to the reference's own GPU-vs-CPU bar:
cosine > 0.999 and max|diff| < 2e-2 * peak.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import bits_of, dev, ok, stream, to_dev

pytestmark = pytest.mark.gpu

HS, NQ, NK, HD, INTER, LAYERS, VOCAB, THETA, EPS = 256, 2, 1, 128, 512, 2, 100, 1e4, 1e-6
T, POS0 = 37, 5


def make_model(seed=2024):
    rng = np.random.default_rng(seed)

    def w(*shape, scale):
        return (rng.standard_normal(shape) * scale).astype(np.float16)

    layers = []
    for _ in range(LAYERS):
        layers.append(dict(
            ln1=(1.0 + 0.1 * rng.standard_normal(HS)).astype(np.float16),
            ln2=(1.0 + 0.1 * rng.standard_normal(HS)).astype(np.float16),
            q=w(NQ * HD, HS, scale=HS ** -0.5), k=w(NK * HD, HS, scale=HS ** -0.5),
            v=w(NK * HD, HS, scale=HS ** -0.5), o=w(HS, NQ * HD, scale=(NQ * HD) ** -0.5),
            qb=w(NQ * HD, scale=0.1), kb=w(NK * HD, scale=0.1),
            gate=w(INTER, HS, scale=HS ** -0.5), up=w(INTER, HS, scale=HS ** -0.5),
            down=w(HS, INTER, scale=INTER ** -0.5)))
    table = w(VOCAB, HS, scale=1.0)
    final = (1.0 + 0.1 * rng.standard_normal(HS)).astype(np.float16)
    ids = rng.integers(0, VOCAB, T).astype(np.int32)
    return table, layers, final, ids


def u16(a):
    return np.ascontiguousarray(a).view(np.uint16)


def dev_attention(q, k, v):
    """Causal GQA on the device in FP32, output FP16 (stand-in, not this library)."""
    qf = q.float().view(T, NQ, HD).transpose(0, 1)
    kf = k.float().view(T, NK, HD).transpose(0, 1).repeat_interleave(NQ // NK, dim=0)
    vf = v.float().view(T, NK, HD).transpose(0, 1).repeat_interleave(NQ // NK, dim=0)
    s = qf @ kf.transpose(1, 2) / HD ** 0.5
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool, device="cuda"), 1), float("-inf"))
    return (torch.softmax(s, -1) @ vf).transpose(0, 1).reshape(T, NQ * HD).half().contiguous()


def linear(x, w):
    """FP16 x [T,in] @ w[out,in]^T with FP32 accumulation, FP16 result (stand-in)."""
    return (x.float() @ w.float().t()).half().contiguous()


def device_chain(table, layers, final, ids, fused):
    st = stream()
    d_table, d_ids = torch.from_numpy(table).cuda(), torch.from_numpy(ids).cuda()
    L = [{k: torch.from_numpy(v).cuda() for k, v in lay.items()} for lay in layers]
    d_final = torch.from_numpy(final).cuda()
    hidden = torch.empty(T, HS, dtype=torch.float16, device="cuda")
    norm_out = torch.empty_like(hidden)
    if fused:
        ok(dev.vv_embedding_rmsnorm_dev(d_table.data_ptr(), d_ids.data_ptr(), L[0]["ln1"].data_ptr(),
                                        hidden.data_ptr(), norm_out.data_ptr(), T, HS, EPS, st))
    else:
        ok(dev.vv_embedding_dev(d_table.data_ptr(), d_ids.data_ptr(), hidden.data_ptr(), T, HS, st))
    for li, w in enumerate(L):
        if not fused:
            ok(dev.vv_rmsnorm_dev(hidden.data_ptr(), w["ln1"].data_ptr(), norm_out.data_ptr(), T, HS,
                                  EPS, st))
        q, k, v = linear(norm_out, w["q"]), linear(norm_out, w["k"]), linear(norm_out, w["v"])
        if fused:
            ok(dev.vv_bias_rope_qk_dev(q.data_ptr(), k.data_ptr(), w["qb"].data_ptr(), w["kb"].data_ptr(),
                                       T, NQ, NK, HD, POS0, None, THETA, st))
        else:
            ok(dev.vv_bias_add_dev(q.data_ptr(), w["qb"].data_ptr(), T, NQ * HD, st))
            ok(dev.vv_bias_add_dev(k.data_ptr(), w["kb"].data_ptr(), T, NK * HD, st))
            ok(dev.vv_rope_dev(q.data_ptr(), T, NQ, HD, POS0, None, THETA, st))
            ok(dev.vv_rope_dev(k.data_ptr(), T, NK, HD, POS0, None, THETA, st))
        attn = dev_attention(q, k, v)
        norm_out.copy_(linear(attn, w["o"]))                 # o_proj writes norm_out (decoder.c:947)
        if fused:
            ok(dev.vv_add_rmsnorm_dev(hidden.data_ptr(), norm_out.data_ptr(), w["ln2"].data_ptr(),
                                      norm_out.data_ptr(), T, HS, EPS, st))
        else:
            ok(dev.vv_residual_add_dev(hidden.data_ptr(), norm_out.data_ptr(), T * HS, st))
            ok(dev.vv_rmsnorm_dev(hidden.data_ptr(), w["ln2"].data_ptr(), norm_out.data_ptr(), T, HS,
                                  EPS, st))
        gate, up = linear(norm_out, w["gate"]), linear(norm_out, w["up"])
        ok(dev.vv_swiglu_dev(gate.data_ptr(), up.data_ptr(), gate.data_ptr(), T * INTER, st))  # in place
        mlp_out = linear(gate, w["down"])
        nxt = L[li + 1]["ln1"] if li + 1 < LAYERS else d_final
        if fused:                                            # residual + the NEXT norm (decoder.c:988 -> :810)
            ok(dev.vv_add_rmsnorm_dev(hidden.data_ptr(), mlp_out.data_ptr(), nxt.data_ptr(),
                                      norm_out.data_ptr(), T, HS, EPS, st))
        else:
            ok(dev.vv_residual_add_dev(hidden.data_ptr(), mlp_out.data_ptr(), T * HS, st))
            if li + 1 == LAYERS:
                ok(dev.vv_rmsnorm_dev(hidden.data_ptr(), d_final.data_ptr(), norm_out.data_ptr(), T, HS,
                                      EPS, st))
    return bits_of(hidden), bits_of(norm_out)


def host_chain(table, layers, final, ids):
    """The CPU path's sequence (decoder_layer_cpu, decoder.c:1332-1484): FP32 activations."""
    def lin(x, w):
        return x @ w.astype(np.float32).T

    hidden = oracle.embedding_f32(u16(table), ids)
    for w in layers:
        n = oracle.rmsnorm_f32(hidden, u16(w["ln1"]), EPS)
        q = lin(n, w["q"]) + w["qb"].astype(np.float32)
        k = lin(n, w["k"]) + w["kb"].astype(np.float32)
        v = lin(n, w["v"])
        q = oracle.rope_f32(q.reshape(T, NQ, HD), POS0, THETA)
        k = oracle.rope_f32(k.reshape(T, NK, HD), POS0, THETA)
        qh = q.transpose(1, 0, 2)
        kh = np.repeat(k.transpose(1, 0, 2), NQ // NK, axis=0)
        vh = np.repeat(v.reshape(T, NK, HD).transpose(1, 0, 2), NQ // NK, axis=0)
        s = qh @ kh.transpose(0, 2, 1) / np.sqrt(HD)
        s = np.where(np.triu(np.ones((T, T), bool), 1)[None], -np.inf, s)
        p = np.exp(s - s.max(-1, keepdims=True))
        attn = ((p / p.sum(-1, keepdims=True)) @ vh).transpose(1, 0, 2).reshape(T, NQ * HD)
        hidden = oracle.residual_add_f32(hidden, lin(attn.astype(np.float32), w["o"]))
        n = oracle.rmsnorm_f32(hidden, u16(w["ln2"]), EPS)
        act = oracle.swiglu_f32(lin(n, w["gate"]), lin(n, w["up"]))
        hidden = oracle.residual_add_f32(hidden, lin(act, w["down"]))
    return hidden, oracle.rmsnorm_f32(hidden, u16(final), EPS)


def test_fused_chain_equals_reference_api_chain_and_matches_cpu():
    table, layers, final, ids = make_model()
    h_ref, n_ref = device_chain(table, layers, final, ids, fused=False)
    h_fus, n_fus = device_chain(table, layers, final, ids, fused=True)
    assert np.array_equal(h_ref, h_fus) and np.array_equal(n_ref, n_fus), \
        "fused entry points changed the bits of the layer chain"

    cpu_h, cpu_n = host_chain(table, layers, final, ids)
    for got_bits, want, what in ((h_ref, cpu_h, "hidden"), (n_ref, cpu_n, "final norm")):
        got = oracle.widen(got_bits).astype(np.float64).ravel()
        want = want.astype(np.float64).ravel()
        cos = float(got @ want / (np.linalg.norm(got) * np.linalg.norm(want)))
        peak = float(np.abs(want).max())
        diff = float(np.abs(got - want).max())
        assert cos > 0.999, f"{what}: cosine {cos}"
        assert diff < 2e-2 * peak, f"{what}: max diff {diff} vs peak {peak}"
