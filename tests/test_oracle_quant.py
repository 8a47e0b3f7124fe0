"""Pins the oracle's int8 activation quantiser (oracle/vv_oracle.c:
vvo_quant_act_q8, vvo_q8_pos) — the checker for vv_act_quant_dev and the fused
*_q8 kernels: against the compiled reference (src/cpu/cpu_int8.c), against a
numpy restatement written from the documented definition, and against the
layouts' descriptions in the reference's q8.h."""
import ctypes as C

import numpy as np
import pytest

import oracle

needs_ref = pytest.mark.skipif(oracle.ref is None or not hasattr(oracle.ref, "vv_quant_act_q8_cpu"),
                               reason="oracle/_ref not built here")


def layout_table(layout):
    return [oracle.lib.vvo_q8_pos(layout, j) for j in range(32)]


def test_layouts_match_their_descriptions():
    """q8.h:19-47 describes each layout in words; build each table from the words."""
    assert layout_table(0) == list(range(32))
    # nibble: the 16 even columns, then the 16 odd ones
    want = [0] * 32
    for n, j in enumerate(list(range(0, 32, 2)) + list(range(1, 32, 2))):
        want[j] = n
    assert layout_table(1) == want
    # W4A16 GPU layout: column j sits in word t = (j/2)%4 at nibble slot s = j/8 + 4*(j%2)
    gemv, mma = [0] * 32, [0] * 32
    for j in range(32):
        t, s = (j // 2) % 4, j // 8 + 4 * (j % 2)
        # GEMV: positions 8t..8t+3 are the even slots (0,2,4,6), 8t+4..8t+7 the odd ones
        gemv[j] = 8 * t + (4 if s % 2 else 0) + s // 2
        # MMA: slots 0..3 of word t at 4t..4t+3, slots 4..7 at 16+4t..16+4t+3
        mma[j] = (16 if s >= 4 else 0) + 4 * t + s % 4
    assert layout_table(2) == gemv and layout_table(3) == mma
    for lay in range(4):
        assert sorted(layout_table(lay)) == list(range(32))       # a permutation


def numpy_quant(x, layout):
    x = x.astype(np.float32)
    amax = np.abs(x).max(axis=1)
    with np.errstate(divide="ignore"):
        inv = np.where(amax > 0, np.float32(127.0) / amax, np.float32(0)).astype(np.float32)
    sx = (amax / np.float32(127.0)).astype(np.float32)
    q = np.clip(np.rint((x * inv[:, None]).astype(np.float32)), -127, 127).astype(np.int32)
    M, K = x.shape
    runs = q.reshape(M, K // 32, 32)
    out = np.empty_like(runs)
    out[:, :, layout_table(layout)] = runs
    return out.reshape(M, K).astype(np.int8), sx, runs.sum(axis=2).astype(np.int32)


@pytest.mark.parametrize("layout", [0, 1, 2, 3])
def test_quantiser_against_numpy_restatement(layout):
    x = oracle.widen(oracle.normal_f16((9, 3584), 11 + layout, std=3.0))
    x[2] = 0.0                                        # zero row: scale 0, all zeros
    x[3, 5] = 1000.0                                  # one outlier sets the scale
    x[4] = np.float32(0.5)                            # ties: 0.5*inv lands on .5 values
    q, sx, xs = oracle.quant_act_q8(x, layout)
    wq, wsx, wxs = numpy_quant(x, layout)
    assert np.array_equal(q, wq) and np.array_equal(sx, wsx) and np.array_equal(xs, wxs)
    assert not q[2].any() and sx[2] == 0.0
    assert np.abs(q.astype(np.int32)).max() == 127 and q.min() >= -127
    # round-half-even, not half-away: 2.5 -> 2, 3.5 -> 4 (amax 127 makes inv exactly 1)
    t = np.zeros((1, 32), np.float32)
    t[0, :5] = [127.0, 2.5, 3.5, -2.5, -0.5]
    tq, _, _ = oracle.quant_act_q8(t, 0)
    assert tq[0, :5].tolist() == [127, 2, 4, -2, 0]


@needs_ref
@pytest.mark.parametrize("M,K", [(1, 32), (7, 1536), (5, 3584), (3, 18944), (2, 22528)])
def test_quantiser_equals_compiled_reference(M, K):
    x = oracle.widen(oracle.normal_f16((M, K), M + K, std=4.0))
    i8p, f32p, i32p = C.POINTER(C.c_int8), C.POINTER(C.c_float), C.POINTER(C.c_int32)
    for layout in range(4):
        q, sx, xs = oracle.quant_act_q8(x, layout)
        rq, rsx, rxs = np.empty_like(q), np.empty_like(sx), np.empty_like(xs)
        assert oracle.ref.vv_quant_act_q8_cpu(x.ctypes.data_as(f32p), M, K, layout, rq.ctypes.data_as(i8p),
                                              rsx.ctypes.data_as(f32p), rxs.ctypes.data_as(i32p)) == 0
        assert np.array_equal(q, rq) and np.array_equal(sx.view(np.uint32), rsx.view(np.uint32))
        assert np.array_equal(xs, rxs)


def test_quantiser_against_golden_vectors():
    import os
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "cpu_kernels_golden.npz"))
    for layout in range(4):
        q, sx, xs = oracle.quant_act_q8(gold["q8_x"], layout)
        assert np.array_equal(q, gold[f"q8_q{layout}"]), layout
        assert np.array_equal(sx.view(np.uint32), gold[f"q8_sx{layout}"].view(np.uint32))
        assert np.array_equal(xs, gold[f"q8_xs{layout}"])


def test_quantiser_argument_checks():
    x = np.zeros((2, 64), np.float32)
    q = np.zeros((2, 64), np.int8)
    sx = np.zeros(2, np.float32)
    i8p, f32p = C.POINTER(C.c_int8), C.POINTER(C.c_float)
    call = oracle.lib.vvo_quant_act_q8
    assert call(x.ctypes.data_as(f32p), 2, 64, 0, q.ctypes.data_as(i8p), sx.ctypes.data_as(f32p), None) == 0
    assert call(x.ctypes.data_as(f32p), 2, 48, 0, q.ctypes.data_as(i8p), sx.ctypes.data_as(f32p), None) == -1
    assert call(x.ctypes.data_as(f32p), 2, 64, 4, q.ctypes.data_as(i8p), sx.ctypes.data_as(f32p), None) == -1
    assert call(None, 2, 64, 0, q.ctypes.data_as(i8p), sx.ctypes.data_as(f32p), None) == -2


def test_w8a8_linear_against_integer_closed_form_and_reference():
    """The int32 dot is exact, so the FP32 output is pinned bit for bit: by the
    compiled reference (vv_w8a8_gemm_cpu) and by an int64 matmul followed by the
    same two FP32 products and one addition."""
    import ctypes as C
    rng = np.random.default_rng(5)
    for M, N, K in ((1, 16, 32), (5, 70, 3584), (9, 33, 160)):
        xq = rng.integers(-127, 128, (M, K), dtype=np.int8)
        w = rng.integers(-127, 128, (N, K), dtype=np.int8)
        sx = rng.uniform(0.001, 0.05, M).astype(np.float32)
        sw = rng.uniform(0.0005, 0.01, N).astype(np.float32)
        bias = oracle.normal_f16((N,), 3, std=0.5)
        res = oracle.normal_f16((M, N), 4)
        t = xq.astype(np.int64) @ w.astype(np.int64).T
        assert np.abs(t).max() < 2 ** 31
        want = (t.astype(np.float32) * sx[:, None]) * sw[None, :]
        plain, _ = oracle.w8a8_linear(xq, sx, w, sw)
        assert np.array_equal(plain, want)
        with_b = want + oracle.widen(bias)[None, :]
        f32, f16 = oracle.w8a8_linear(xq, sx, w, sw, bias, res)
        assert np.array_equal(f32, with_b + oracle.widen(res))
        assert np.array_equal(f16, f32.astype(np.float16).view(np.uint16))
        if oracle.ref is not None and hasattr(oracle.ref, "vv_w8a8_gemm_cpu"):
            out = np.empty((M, N), np.float32)
            f32p = C.POINTER(C.c_float)
            assert oracle.ref.vv_w8a8_gemm_cpu(xq.ctypes.data, sx.ctypes.data_as(f32p), w.ctypes.data,
                                               sw.ctypes.data_as(f32p), bias.ctypes.data,
                                               out.ctypes.data_as(f32p), M, N, K) == 0
            assert np.array_equal(out, with_b)


def int4_problem(N, K, G, seed, unit=False):
    rng = np.random.default_rng(seed)
    packed = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    zeros = rng.integers(0, 16, (N, K // G), dtype=np.uint8)
    if unit:
        scales = np.full((N, K // G), 0x3C00, np.uint16)
    else:
        scales = rng.uniform(0.002, 0.022, (N, K // G)).astype(np.float16).view(np.uint16)
    return packed, scales, zeros


def int4_codes(packed):
    """[N,K/2] row-major INT4G bytes -> [N,K] codes (high nibble = even column)."""
    out = np.empty((packed.shape[0], packed.shape[1] * 2), np.int64)
    out[:, 0::2], out[:, 1::2] = packed >> 4, packed & 15
    return out


def test_w4a8_linear_against_closed_form_and_reference():
    """Integer part: an int64 matmul of (q - z) per group. With unit scales the
    FP32 output is that integer exactly (and so is the compiled reference's,
    whichever instruction set it picked); with real scales the groups are
    added in order in FP32, checked against float64 to the worst case of that
    many roundings ((groups + 2) * 2^-24 of the sum of magnitudes). The
    compiled reference's vector kernels scale partial sums of q x and z x
    separately, so they agree to the same count of roundings of THOSE
    magnitudes (sum_k s (q + z) |x|), no closer."""
    import ctypes as C
    rng = np.random.default_rng(8)
    f32p, i32p = C.POINTER(C.c_float), C.POINTER(C.c_int32)
    for M, N, K, G in ((1, 16, 64, 32), (5, 40, 3584, 128), (9, 33, 1024, 512), (4, 24, 256, 256)):
        x = rng.normal(size=(M, K)).astype(np.float32) * 3
        xq, sx, xs = oracle.quant_act_q8(x, 0)
        xq_nib, _, _ = oracle.quant_act_q8(x, 1)
        ng = K // G
        for unit in (True, False):
            packed, scales, zeros = int4_problem(N, K, G, 11 + N, unit)
            d = int4_codes(packed).reshape(N, ng, G) - zeros[:, :, None].astype(np.int64)
            per_group = np.einsum("mgk,ngk->mng", xq.astype(np.int64).reshape(M, ng, G), d)
            s = oracle.widen(scales).astype(np.float64)
            one = np.ones(M, np.float32)
            got, _ = oracle.w4a8_linear(xq, one if unit else sx, packed, scales, zeros, G)
            exact = (per_group * s[None]).sum(-1) * (1.0 if unit else sx[:, None].astype(np.float64))
            mag = (np.abs(per_group) * s[None]).sum(-1) * (1.0 if unit else sx[:, None])
            bar = (ng + 2) * 2.0 ** -24 * mag + 1e-30
            if unit:
                assert np.abs(exact).max() < 2 ** 24 and np.array_equal(got.astype(np.float64), exact)
            else:
                assert np.max(np.abs(got - exact) / bar) <= 1.0
            if oracle.ref is not None and hasattr(oracle.ref, "vv_w4a8_gemm_cpu"):
                out = np.empty((M, N), np.float32)
                sxu = one if unit else sx
                assert oracle.ref.vv_w4a8_gemm_cpu(xq_nib.ctypes.data, sxu.ctypes.data_as(f32p),
                                                   xs.ctypes.data_as(i32p), packed.ctypes.data, scales.ctypes.data,
                                                   zeros.ctypes.data, G, None, out.ctypes.data_as(f32p),
                                                   M, N, K) == 0
                if unit:
                    assert np.array_equal(out, got)
                else:
                    qz = int4_codes(packed).reshape(N, ng, G) + zeros[:, :, None].astype(np.int64)
                    loose = np.einsum("mgk,ngk->mng", np.abs(xq.astype(np.int64)).reshape(M, ng, G), qz)
                    loose = (loose * s[None]).sum(-1) * sx[:, None]
                    assert np.max(np.abs(out - got) / ((ng + 2) * 2.0 ** -24 * loose)) <= 1.0
        bias = oracle.normal_f16((N,), 3, std=0.5)
        res = oracle.normal_f16((M, N), 4)
        plain, _ = oracle.w4a8_linear(xq, sx, packed, scales, zeros, G)
        f32, f16 = oracle.w4a8_linear(xq, sx, packed, scales, zeros, G, bias, res)
        assert np.array_equal(f32, (plain + oracle.widen(bias)[None, :]) + oracle.widen(res))
        assert np.array_equal(f16, f32.astype(np.float16).view(np.uint16))


def test_int4_gpu_layout_against_reference_and_the_activation_orders():
    """The converter against the compiled reference byte for byte, and against
    what the layout is for: reading word t of a chunk as `w & 0x0F0F0F0F` /
    `(w >> 4) & 0x0F0F0F0F` next to activations in VV_Q8_W4_GEMV order, or as
    its low / high 16 bits next to VV_Q8_W4_MMA order, gives the same integer
    dot as codes and activations both in column order."""
    N, K, G = 12, 256, 64
    packed, scales, zeros = int4_problem(N, K, G, 2)
    gpu, sz = oracle.int4g_to_gpu_layout(packed, scales, zeros, G)
    assert np.array_equal(sz[:, :, 0], scales)
    assert np.array_equal(oracle.widen(sz[:, :, 1]), zeros.astype(np.float32))
    if oracle.ref is not None and hasattr(oracle.ref, "vv_int4g_to_gpu_layout"):
        theirs, their_sz = packed.copy(), np.empty_like(sz)
        assert oracle.ref.vv_int4g_to_gpu_layout(theirs.ctypes.data, scales.ctypes.data, zeros.ctypes.data,
                                                 N, K, G, their_sz.ctypes.data) == 0
        assert np.array_equal(theirs, gpu) and np.array_equal(their_sz, sz)
    x = np.random.default_rng(3).normal(size=(3, K)).astype(np.float32)
    nat, _, _ = oracle.quant_act_q8(x, 0)
    gemv, _, _ = oracle.quant_act_q8(x, 2)
    mma, _, _ = oracle.quant_act_q8(x, 3)
    want = nat.astype(np.int64) @ int4_codes(packed).T
    words = gpu.reshape(N, K // 32, 4, 4).astype(np.uint32)
    words = words[..., 0] | words[..., 1] << 8 | words[..., 2] << 16 | words[..., 3] << 24      # [N, chunk, t]
    nib = np.stack([(words >> (4 * s)) & 15 for s in range(8)], axis=-1).astype(np.int64)    # [N, chunk, t, slot]
    # GEMV order: positions 8t..8t+3 meet slots 0,2,4,6 and 8t+4..8t+7 slots 1,3,5,7
    by_gemv = np.concatenate([nib[..., 0::2], nib[..., 1::2]], axis=-1).reshape(N, K)
    assert np.array_equal(gemv.astype(np.int64) @ by_gemv.T, want)
    # MMA order: positions 4t..4t+3 meet slots 0..3, positions 16+4t.. slots 4..7
    by_mma = np.concatenate([nib[..., :4].reshape(N, K // 32, 16), nib[..., 4:].reshape(N, K // 32, 16)],
                            axis=-1).reshape(N, K)
    assert np.array_equal(mma.astype(np.int64) @ by_mma.T, want)


def test_int4_dequant_against_closed_form_and_reference_gemm():
    """(q - z) * s: the FP64 product is exact, so its direct rounding to FP16
    pins every bit. The compiled reference's CPU GEMM dequantises as
    q * s + fp16(-z * s) (one more rounding per weight), so a product of these
    weights agrees with it to FP16 weight precision, not bit for bit."""
    import ctypes as C
    N, K, G, M = 24, 256, 64, 5
    packed, scales, zeros = int4_problem(N, K, G, 4)
    w16 = oracle.int4g_dequant_f16(packed, scales, zeros, G)
    d = int4_codes(packed) - np.repeat(zeros.astype(np.int64), G, axis=1)
    s = np.repeat(oracle.widen(scales).astype(np.float64), G, axis=1)
    assert np.array_equal(w16, (d * s).astype(np.float16).view(np.uint16))
    if oracle.ref is not None and hasattr(oracle.ref, "vv_int4g_gemm_cpu"):
        x = np.random.default_rng(6).normal(size=(M, K)).astype(np.float32)
        mins = (-(zeros.astype(np.float32)) * oracle.widen(scales)).astype(np.float16).view(np.uint16)
        out = np.empty((M, N), np.float32)
        f32p = C.POINTER(C.c_float)
        assert oracle.ref.vv_int4g_gemm_cpu(x.ctypes.data_as(f32p), packed.ctypes.data, scales.ctypes.data,
                                            mins.ctypes.data, None, out.ctypes.data_as(f32p), M, N, K, G) == 0
        ours = oracle.gemm_f16w(x, w16)
        mag = np.abs(x).astype(np.float64) @ np.abs(oracle.widen(w16)).astype(np.float64).T
        assert np.max(np.abs(out - ours) / mag) < 2e-3


# ── the older weight-only formats ───────────────────────────────────────────

def _identity_through(fn, K, N, *weights):
    """Push the identity through a CPU GEMM of the compiled reference: row m of the
    output is column m of the weight it multiplies, with nothing added to it."""
    eye = np.eye(K, dtype=np.float32)
    out = np.empty((K, N), np.float32)
    fp = C.POINTER(C.c_float)
    rc = fn(eye.ctypes.data_as(fp), *weights, None, out.ctypes.data_as(fp), K, N, K)
    assert rc == 0
    return out.T


def test_weight_only_dequantisers_against_closed_forms():
    rng = np.random.default_rng(5)
    N, K = 12, 256
    # NF4: every code against the published code book, high nibble first, one absmax per 64 flat elements
    book = np.array([-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
                     -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
                     0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
                     0.7229568362236023, 1.0], np.float32)
    assert np.all(np.diff(book) > 0) and book[7] == 0.0
    p = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    s = oracle.narrow(rng.uniform(0.01, 0.3, N * K // 64).astype(np.float32))
    w16, w32 = oracle.nf4_dequant(p, s)
    codes = np.stack([p >> 4, p & 15], -1).reshape(N, K)
    want = book[codes] * np.repeat(oracle.widen(s), 64).reshape(N, K)
    assert np.array_equal(w32, want.astype(np.float32))
    assert np.array_equal(w16, want.astype(np.float32).astype(np.float16).view(np.uint16))
    # INT4 {scale, min}: q * s + m is exact in FP64, one rounding to FP32 and one to FP16
    G = 64
    sc = oracle.narrow(rng.uniform(0.01, 0.05, (N, K // G)).astype(np.float32))
    mn = oracle.narrow(-rng.uniform(0.05, 0.4, (N, K // G)).astype(np.float32))
    w16, w32 = oracle.awq_dequant(p, sc, mn, G)
    exact = codes.astype(np.float64) * np.repeat(oracle.widen(sc).astype(np.float64), G, 1) \
        + np.repeat(oracle.widen(mn).astype(np.float64), G, 1)
    assert np.array_equal(w32, exact.astype(np.float32))
    assert np.array_equal(w16, exact.astype(np.float32).astype(np.float16).view(np.uint16))
    # INT8: the FP32 product, then FP16
    q = rng.integers(-128, 128, (N, K), dtype=np.int8)
    s8 = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    w16, w32 = oracle.int8_dequant(q, s8)
    want = q.astype(np.float32) * s8[:, None]
    assert np.array_equal(w32, want) and np.array_equal(w16, want.astype(np.float16).view(np.uint16))


@pytest.mark.skipif(oracle.ref is None or not hasattr(oracle.ref, "vv_nf4_gemm_cpu"),
                    reason="oracle/_ref not built (needs the reference tree)")
def test_weight_only_dequantisers_against_the_compiled_reference():
    """The reference's CPU kernels multiply the FP32 weight: the identity pushed
    through them must return the oracle's FP32 weights exactly."""
    rng = np.random.default_rng(6)
    N, K, G = 24, 256, 64
    p = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    s = oracle.narrow(rng.uniform(0.01, 0.3, N * K // 64).astype(np.float32))
    assert np.array_equal(_identity_through(oracle.ref.vv_nf4_gemm_cpu, K, N, p.ctypes.data, s.ctypes.data),
                          oracle.nf4_dequant(p, s)[1])
    q = rng.integers(-128, 128, (N, K), dtype=np.int8)
    s8 = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    assert np.array_equal(_identity_through(oracle.ref.vv_int8_gemm_cpu, K, N, q.ctypes.data, s8.ctypes.data),
                          oracle.int8_dequant(q, s8)[1])
    sc = oracle.narrow(rng.uniform(0.01, 0.05, (N, K // G)).astype(np.float32))
    mn = oracle.narrow(-rng.uniform(0.05, 0.4, (N, K // G)).astype(np.float32))
    eye = np.eye(K, dtype=np.float32)
    out = np.empty((K, N), np.float32)
    fp = C.POINTER(C.c_float)
    assert oracle.ref.vv_int4g_gemm_cpu(eye.ctypes.data_as(fp), p.ctypes.data, sc.ctypes.data, mn.ctypes.data, None,
                                        out.ctypes.data_as(fp), K, N, K, G) == 0
    assert np.array_equal(out.T, oracle.awq_dequant(p, sc, mn, G)[1])
