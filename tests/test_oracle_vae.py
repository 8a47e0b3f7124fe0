"""CPU checks of the oracle's Conv-VAE restatement. The reference's CPU encoder
works in FP32 with other roundings, so these functions are pinned by what the
mathematics fixes: numpy convolutions in FP64 (to the FP32 chain's rounding and
one FP16 rounding), invariance under chunking (bit for bit), im2col + GEMM ==
direct conv (bit for bit), closed forms for the statistics and epilogues, and an
exhaustive check of the truncating FP16 conversion."""
import numpy as np
import pytest

import oracle
from oracle import VaeConvDesc, VaeRows


def f16(shape, seed, std=1.0):
    return oracle.normal_f16(shape, seed, std=std)


def W(a):
    return oracle.widen(a).astype(np.float64)


def one_item(in_len, out_len, have=0, keep=0, cap=0, tail_in=None, tail_out=None, in_off=0, out_off=0):
    d = VaeConvDesc()
    d.n, d.cap = 1, cap
    it = d.it[0]
    it.in_off, it.out_off, it.in_len, it.out_len, it.have, it.keep = in_off, out_off, in_len, out_len, have, keep
    it.tail_in = tail_in.ctypes.data if tail_in is not None else None
    it.tail_out = tail_out.ctypes.data if tail_out is not None else None
    return d


def conv_whole(x, w, b, k, stride, out_len, pad_left):
    """FP64 causal conv with pad_left zero columns in front of x [in_ch, T]."""
    in_ch, T = x.shape
    xp = np.concatenate([np.zeros((in_ch, pad_left)), W(x), np.zeros((in_ch, k * stride + stride))], 1)
    out = np.zeros((w.shape[0], out_len))
    for t in range(out_len):
        out[:, t] = np.einsum("oik,ik->o", W(w), xp[:, t * stride:t * stride + k])
    return out + (W(b)[:, None] if b is not None else 0.0)


@pytest.mark.parametrize("in_ch,out_ch,k,stride", [(1, 8, 7, 1), (8, 16, 4, 2), (16, 12, 6, 3)])
def test_conv_matches_fp64_and_chunking_changes_no_bit(in_ch, out_ch, k, stride):
    T = 120 * stride
    x, w, b = f16((in_ch, T), 1), f16((out_ch, in_ch, k), 2, std=(in_ch * k) ** -0.5), f16((out_ch,), 3, std=0.2)
    ctx = k - stride                                  # the columns a causal conv of this stride looks back over
    out_len = T // stride
    # whole signal, fresh state: `have` zero-context columns
    zeros = np.zeros((in_ch, ctx), np.uint16)
    d = one_item(T, out_len, have=ctx, cap=ctx, tail_in=zeros if ctx else None)
    y = np.zeros((out_ch, out_len), np.uint16)
    oracle.vae_conv(d, x, T, w, b, y, out_len, in_ch, out_ch, k, stride)
    ref = conv_whole(x, w, b, k, stride, out_len, ctx)
    mag = conv_whole(oracle.narrow(np.abs(oracle.widen(x))), oracle.narrow(np.abs(oracle.widen(w))), None, k, stride,
                     out_len, ctx)
    ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(W(y) - ref) <= 0.5 * ulp + in_ch * k * 2.0 ** -24 * mag + 1e-7)
    # the same signal in three ragged chunks, the state carried through vae_tail: the same bits
    cuts = [0, 37 * stride, 38 * stride, T]
    state = zeros.copy() if ctx else None
    got = np.zeros_like(y)
    for a, e in zip(cuts[:-1], cuts[1:]):
        n_in, n_out = e - a, (e - a) // stride
        nxt = np.zeros_like(state) if ctx else None
        chunk = np.ascontiguousarray(x[:, a:e])
        dc = one_item(n_in, n_out, have=ctx, keep=ctx, cap=ctx, tail_in=state, tail_out=nxt)
        part = np.zeros((out_ch, n_out), np.uint16)
        oracle.vae_conv(dc, chunk, n_in, w, b, part, n_out, in_ch, out_ch, k, stride)
        oracle.vae_tail(dc, chunk, n_in, in_ch)
        got[:, a // stride:e // stride] = part
        state = nxt
    assert np.array_equal(got, y)
    # im2col + the GEMM over its columns: the same bits again
    col = np.zeros((in_ch * k, out_len), np.uint16)
    oracle.vae_im2col(d, x, T, in_ch, k, stride, 0, out_len, col, out_len)
    assert np.array_equal(col.reshape(in_ch, k, out_len)[:, 0, 1], np.concatenate([zeros, x], 1)[:, stride])
    y2 = np.zeros_like(y)
    oracle.vae_conv_gemm(w, col, out_len, b, y2, out_len, out_ch, in_ch * k, out_len)
    assert np.array_equal(y2, y)
    # transposed output with skipped frames
    yt = np.zeros((out_len - 2, out_ch + 3), np.uint16)
    d.it[0].out_ptr, d.it[0].out_ld, d.it[0].skip = yt.ctypes.data, out_ch + 3, 2
    oracle.vae_conv(d, x, T, w, b, None, 0, in_ch, out_ch, k, stride, transposed=True)
    assert np.array_equal(yt[:, :out_ch], y[:, 2:].T) and not yt[:, out_ch:].any()


def test_rms_and_mixer_closed_forms():
    C, T, k = 24, 90, 7
    x = f16((C, T), 5)
    tail = f16((C, k - 1), 6)
    d = one_item(T, T, have=k - 1, cap=k - 1, tail_in=tail)
    rinv = np.zeros(T + (k - 1), np.float32)
    oracle.vae_rms(x, T, T, C, 1e-5, rinv, d)
    want = 1.0 / np.sqrt((W(np.concatenate([x, tail], 1)) ** 2).mean(0) + 1e-5)
    assert np.allclose(rinv, want, rtol=3e-7 * C ** 0.5, atol=0)
    nw, cw, cb, g = f16((C,), 7, std=0.5), f16((C, k), 8, std=0.4), f16((C,), 9, std=0.1), f16((C,), 10, std=0.3)
    out = np.zeros_like(x)
    oracle.vae_mixer(d, x, out, T, rinv, T, nw, cw, cb, g, C, k)
    full = np.concatenate([tail, x], 1)
    normed = W(full) * np.concatenate([want[T:], want[:T]])[None, :] * W(nw)[:, None]
    normed = normed.astype(np.float16).astype(np.float64)                       # the stored intermediate
    y = np.stack([(normed[:, t:t + k] * W(cw)).sum(1) for t in range(T)], 1) + W(cb)[:, None]
    ref = W(x) + y * W(g)[:, None]
    err = np.abs(W(out) - ref)
    assert err.max() <= 2e-3 * np.abs(ref).max() and (err > 1.5 * np.spacing(np.abs(ref).astype(np.float16))).mean() < 0.01
    # without a state the left halo is zeros
    d0 = one_item(T, T)
    out0 = np.zeros_like(x)
    oracle.vae_mixer(d0, x, out0, T, rinv, T, nw, cw, cb, None, C, k)
    normed0 = np.concatenate([np.zeros((C, k - 1)), normed[:, k - 1:]], 1)
    y0 = np.stack([(normed0[:, t:t + k] * W(cw)).sum(1) for t in range(T)], 1) + W(cb)[:, None]
    assert np.abs(W(out0) - (W(x) + y0)).max() <= 2e-3 * np.abs(ref).max()


@pytest.mark.parametrize("epi", [0, 1, 2])
def test_gemm_nn_epilogues(epi):
    from scipy.special import erf
    M, K, P, ldb, ldc = 20, 48, 70, 75, 72
    A, B = f16((M, K), 11, std=K ** -0.5), f16((K, ldb), 12)
    bias, gamma = f16((M,), 13, std=0.3), f16((M,), 14, std=0.5)
    Cm = f16((M, ldc), 15)
    keep = Cm.copy()
    rinv = np.random.default_rng(16).uniform(0.5, 1.5, ldb).astype(np.float32)
    nw = f16((K,), 17, std=0.7)
    oracle.vae_gemm_nn(epi, A, B, ldb, Cm, ldc, M, K, P, bias, gamma, rinv, nw)
    Bn = (W(B) * rinv[None, :] * W(nw)[:, None]).astype(np.float16).astype(np.float64)
    acc = W(A) @ Bn[:, :P]
    if epi == 2:
        ref = acc + W(bias)[:, None]
    else:
        v = (acc.astype(np.float16).astype(np.float64) + W(bias)[:, None]).astype(np.float16).astype(np.float64)
        ref = 0.5 * v * (1 + erf(v / np.sqrt(2))) if epi == 0 else W(keep)[:, :P] + v * W(gamma)[:, None]
    got = W(Cm)[:, :P]
    assert np.abs(got - ref).max() <= 1.5e-3 * np.abs(ref).max()
    assert np.array_equal(Cm[:, P:], keep[:, P:])                 # nothing past the window


def test_gemm_tn_rows_and_truncation():
    M, N, K, lda = 12, 10, 32, 40
    A, B, bias = f16((M, lda), 21, std=K ** -0.5), f16((N, K), 22), f16((N,), 23, std=0.2)
    plain = np.zeros((M, N), np.uint16)
    oracle.vae_gemm_tn(A, lda, B, plain, N, M, N, K, bias)
    ref = W(A)[:, :K] @ W(B).T + W(bias)[None, :]
    assert np.abs(W(plain) - ref).max() <= 2e-3 * np.abs(ref).max()
    rows = VaeRows()
    a, b = np.zeros((5, N + 2), np.uint16), np.zeros((7, N), np.uint16)
    rows.mode, rows.n = 1, 2
    rows.seg[0].row0, rows.seg[0].ld, rows.seg[0].dst = 0, N + 2, a.ctypes.data
    rows.seg[1].row0, rows.seg[1].ld, rows.seg[1].dst = 5, N, b.ctypes.data
    oracle.vae_gemm_tn(A, lda, B, None, 0, M, N, K, bias, rows)
    assert np.array_equal(a[:, :N], plain[:5]) and np.array_equal(b, plain[5:]) and not a[:, N:].any()
    rows.mode = 3                                                  # accumulate on top, truncating
    oracle.vae_gemm_tn(A, lda, B, None, 0, M, N, K, bias, rows)
    want = np.array([oracle.trunc_half(2.0 * v) for v in oracle.widen(plain[5:]).ravel()], np.uint16).reshape(7, N)
    assert np.array_equal(b, want)


def test_truncating_conversion_exhaustive_over_fp16_and_edges():
    """Every FP16 value widened to FP32 comes back unchanged unless it is subnormal (flushed to a signed zero); values
    between two FP16 neighbours go to the one nearer zero; past the range to infinity."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    vals = oracle.widen(bits)
    for b, v in zip(bits[::7], vals[::7]):
        if np.isnan(v):
            continue
        want = int(b) if (b & 0x7C00) != 0 else int(b & 0x8000)
        assert oracle.trunc_half(float(v)) == want
    assert oracle.trunc_half(1.0 + 2.0 ** -11 + 2.0 ** -12) == 0x3C00          # truncates, does not round up
    assert oracle.trunc_half(-(1.0 + 1023.9 / 1024)) == 0xBFFF
    assert oracle.trunc_half(65520.0) == 0x7BFF and oracle.trunc_half(65536.0) == 0x7C00
    assert oracle.trunc_half(6.0e-5) == 0x0000 and oracle.trunc_half(-6.0e-5) == 0x8000
