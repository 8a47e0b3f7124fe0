"""GPU parity tests: every layer op of libvibevoice_hip.so, called through the
C ABI, against the CPU oracle on the same seeded FP16 inputs.

Bars (written where they are applied, in gpu_util.assert_fp16_close):
  * embedding gather, residual add, bias add, the updated residual of the
    fused add+norm, and FP16<->FP32 conversion: BIT-EXACT;
  * RMSNorm, RoPE, SwiGLU outputs (FP16): max|err| / max|ref| <= 2e-3, and on
    top of that at most 1 FP16 ulp from the oracle's correctly rounded value.
Shapes are the benchmark's configurations 2-5 plus the generic widths the reference's own
tests and callers use (tests/test_int8_linear.c:297, test_prefill_append.c:30).
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import assert_fp16_close, assert_rope_close, bits_of, dev, ok, stream, to_dev

pytestmark = pytest.mark.gpu

H, I_FF, V, NQ, NK, HD = 3584, 18944, 152064, 28, 4, 128
EPS = 1e-6


def weight(n, seed=99):
    return oracle.normal_f16((n,), seed, mean=1.0, std=0.1)


# ── RMSNorm ─────────────────────────────────────────────────────────────────

@pytest.mark.parametrize("rows", [1, 7, 512, 4096])
def test_rmsnorm_qwen_width(rows):
    x, w = oracle.normal_f16((rows, H), 100 + rows), weight(H)
    d_x, d_w = to_dev(x), to_dev(w)
    d_y = torch.empty_like(d_x)
    ok(dev.vv_rmsnorm_dev(d_x.data_ptr(), d_w.data_ptr(), d_y.data_ptr(), rows, H, EPS, stream()))
    ref, rne = oracle.rmsnorm_f16(x, w, EPS)
    assert_fp16_close(bits_of(d_y), ref, rne, f"rmsnorm T={rows}")
    assert np.array_equal(bits_of(d_x), x)          # the input is left alone


@pytest.mark.parametrize("hidden", [8, 100, 130, 256, 1536, 2048, 3072, 4096, 8960, 18944])
@pytest.mark.parametrize("rows", [1, 7, 285])
def test_rmsnorm_other_widths(rows, hidden):
    """Every width the reference's callers and tests use, plus widths that are
    not a multiple of 8 (2-byte path) and partial last chunks."""
    x = oracle.normal_f16((rows, hidden), 7 * hidden + rows, std=3.0)
    w = oracle.normal_f16((hidden,), 5, mean=0.5, std=0.25)
    d_x, d_w = to_dev(x), to_dev(w)
    d_y = torch.empty_like(d_x)
    ok(dev.vv_rmsnorm_dev(d_x.data_ptr(), d_w.data_ptr(), d_y.data_ptr(), rows, hidden, EPS,
                          stream()))
    ref, rne = oracle.rmsnorm_f16(x, w, EPS)
    assert_fp16_close(bits_of(d_y), ref, rne, f"rmsnorm [{rows},{hidden}]")


def test_rmsnorm_unaligned_pointers_and_special_rows():
    rows = 5
    x = oracle.normal_f16((rows, H), 11)
    x[1] = 0                                   # zero row -> zero output
    x[2] = oracle.narrow(np.full(H, -2.5, np.float32))   # constant row -> -w
    x[3] = oracle.narrow(oracle.widen(x[3]) * np.float32(2.0 ** -12))   # eps-dominated
    w = weight(H)
    ref, rne = oracle.rmsnorm_f16(x, w, EPS)
    # offset every buffer by one half: 2-byte aligned only
    flat_x = torch.zeros(rows * H + 8, dtype=torch.float16, device="cuda")
    flat_w = torch.zeros(H + 8, dtype=torch.float16, device="cuda")
    flat_y = torch.zeros(rows * H + 8, dtype=torch.float16, device="cuda")
    flat_x[1:1 + rows * H] = to_dev(x).reshape(-1)
    flat_w[1:1 + H] = to_dev(w)
    ok(dev.vv_rmsnorm_dev(flat_x.data_ptr() + 2, flat_w.data_ptr() + 2, flat_y.data_ptr() + 2,
                          rows, H, EPS, stream()))
    got = bits_of(flat_y)
    assert got[0] == 0 and not got[1 + rows * H:].any()        # nothing written outside
    got = got[1:1 + rows * H].reshape(rows, H)
    assert_fp16_close(got, ref, rne, "rmsnorm unaligned")
    assert not got[1].any()
    # aligned call gives the same bits as the unaligned one
    d_x, d_w = to_dev(x), to_dev(w)
    d_y = torch.empty_like(d_x)
    ok(dev.vv_rmsnorm_dev(d_x.data_ptr(), d_w.data_ptr(), d_y.data_ptr(), rows, H, EPS, stream()))
    assert_fp16_close(bits_of(d_y), ref, rne, "rmsnorm aligned")


# ── residual add, fused add + RMSNorm (config 2) ────────────────────────────

def test_residual_add_bit_exact_all_value_classes():
    rng = np.random.default_rng(3)
    n = 1_000_003                                # odd: vector body + 2-byte tail
    a = rng.integers(0, 65536, n, dtype=np.uint16)
    b = rng.integers(0, 65536, n, dtype=np.uint16)
    a[:6] = [0x0000, 0x8000, 0x0001, 0x7BFF, 0x7BFF, 0x7C00]
    b[:6] = [0x8000, 0x8000, 0x8001, 0x7BFF, 0x0001, 0xFC00]
    want = oracle.residual_add_f16(a, b)
    d_a, d_b = to_dev(a), to_dev(b)
    ok(dev.vv_residual_add_dev(d_a.data_ptr(), d_b.data_ptr(), n, stream()))
    got = bits_of(d_a)
    nan = np.isnan(want.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(got.view(np.float16)[nan]).all()
    assert np.array_equal(bits_of(d_b), b)
    # 2-byte aligned buffers take the scalar kernel and give the same bits
    fa = torch.zeros(n + 8, dtype=torch.float16, device="cuda")
    fa[1:1 + n] = to_dev(a)
    ok(dev.vv_residual_add_dev(fa.data_ptr() + 2, d_b.data_ptr(), n, stream()))
    got2 = bits_of(fa)
    assert got2[0] == 0 and not got2[1 + n:].any()
    assert np.array_equal(got2[1:1 + n][~nan], want[~nan])


@pytest.mark.parametrize("rows", [1, 512, 4096])
def test_add_rmsnorm_config2(rows):
    res = oracle.normal_f16((rows, H), 200 + rows)
    x = oracle.normal_f16((rows, H), 300 + rows)
    w = weight(H)
    want_res, nref, nrne = oracle.add_rmsnorm_f16(res, x, w, EPS)
    d_res, d_x, d_w = to_dev(res), to_dev(x), to_dev(w)
    d_n = torch.empty_like(d_res)
    ok(dev.vv_add_rmsnorm_dev(d_res.data_ptr(), d_x.data_ptr(), d_w.data_ptr(), d_n.data_ptr(),
                              rows, H, EPS, stream()))
    assert np.array_equal(bits_of(d_res), want_res), "updated residual must be bit-exact"
    assert_fp16_close(bits_of(d_n), nref, nrne, f"add+rmsnorm T={rows}")
    assert np.array_equal(bits_of(d_x), x)

    # drop-in equivalence: the fused call == residual_add then rmsnorm, bit for bit,
    # with the norm writing over the branch output as the decoder does (decoder.c:950-960)
    e_res, e_x = to_dev(res), to_dev(x)
    ok(dev.vv_residual_add_dev(e_res.data_ptr(), e_x.data_ptr(), rows * H, stream()))
    ok(dev.vv_rmsnorm_dev(e_res.data_ptr(), d_w.data_ptr(), e_x.data_ptr(), rows, H, EPS, stream()))
    assert np.array_equal(bits_of(e_res), bits_of(d_res))
    assert np.array_equal(bits_of(e_x), bits_of(d_n))
    # and the fused call may write `normed` over `x` too
    f_res, f_x = to_dev(res), to_dev(x)
    ok(dev.vv_add_rmsnorm_dev(f_res.data_ptr(), f_x.data_ptr(), d_w.data_ptr(), f_x.data_ptr(),
                              rows, H, EPS, stream()))
    assert np.array_equal(bits_of(f_x), bits_of(d_n))
    assert np.array_equal(bits_of(f_res), want_res)


@pytest.mark.parametrize("rows,hidden", [(3, 100), (9, 1536), (2, 8960), (4, 130)])
def test_add_rmsnorm_other_widths(rows, hidden):
    res = oracle.normal_f16((rows, hidden), 1)
    x = oracle.normal_f16((rows, hidden), 2)
    w = weight(hidden)
    want_res, nref, nrne = oracle.add_rmsnorm_f16(res, x, w, EPS)
    d_res, d_x, d_w = to_dev(res), to_dev(x), to_dev(w)
    d_n = torch.empty_like(d_res)
    ok(dev.vv_add_rmsnorm_dev(d_res.data_ptr(), d_x.data_ptr(), d_w.data_ptr(), d_n.data_ptr(),
                              rows, hidden, EPS, stream()))
    assert np.array_equal(bits_of(d_res), want_res)
    assert_fp16_close(bits_of(d_n), nref, nrne, f"add+rmsnorm [{rows},{hidden}]")


@pytest.mark.parametrize("rows,hidden", [(900, 3584), (1000, 3584), (2049, 3584), (5000, 3584), (3000, 1536),
                                         (4001, 1000), (1300, 4096), (9000, 512)])
def test_mid_size_launches_every_row_kernel_agrees(rows, hidden):
    """Launches of a thousand to a few thousand rows run one wave per row (full and partial
    last groups of 64 chunks), shorter and longer ones a workgroup per row or per two rows, and
    the switch-over differs by op: the fused ops must still equal their two-call sequences bit
    for bit, whichever kernels the two sides run, and both must match the oracle."""
    res = oracle.normal_f16((rows, hidden), 21 + rows)
    x = oracle.normal_f16((rows, hidden), 22 + rows)
    w = weight(hidden)
    want_res, nref, nrne = oracle.add_rmsnorm_f16(res, x, w, EPS)
    d_res, d_x, d_w = to_dev(res), to_dev(x), to_dev(w)
    d_n = torch.full((rows, hidden), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_add_rmsnorm_dev(d_res.data_ptr(), d_x.data_ptr(), d_w.data_ptr(), d_n.data_ptr(),
                              rows, hidden, EPS, stream()))
    assert np.array_equal(bits_of(d_res), want_res), "updated residual must be bit-exact"
    assert_fp16_close(bits_of(d_n), nref, nrne, f"add+rmsnorm [{rows},{hidden}]")
    e_res, e_x = to_dev(res), to_dev(x)
    ok(dev.vv_residual_add_dev(e_res.data_ptr(), e_x.data_ptr(), rows * hidden, stream()))
    ok(dev.vv_rmsnorm_dev(e_res.data_ptr(), d_w.data_ptr(), e_x.data_ptr(), rows, hidden, EPS, stream()))
    assert np.array_equal(bits_of(e_res), bits_of(d_res))
    assert np.array_equal(bits_of(e_x), bits_of(d_n))
    # a row normalised alone (one-row launch: workgroup kernel) gives the bits it got in the batch
    for r in (0, rows // 2, rows - 1):
        one = torch.empty(hidden, dtype=torch.float16, device="cuda")
        ok(dev.vv_rmsnorm_dev(d_res.data_ptr() + r * hidden * 2, d_w.data_ptr(), one.data_ptr(), 1, hidden,
                              EPS, stream()))
        assert np.array_equal(bits_of(one), bits_of(d_n)[r])
    # gather + norm against gather, then norm
    vocab = 3000
    table = oracle.normal_f16((vocab, hidden), 23, std=0.02)
    ids = oracle.ids(rows, 24 + rows, vocab)
    ids[0], ids[-1] = vocab - 1, 0
    d_t, d_i = to_dev(table), torch.from_numpy(ids).cuda()
    g_h = torch.full((rows, hidden), float("nan"), dtype=torch.float16, device="cuda")
    g_n = torch.full((rows, hidden), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_embedding_rmsnorm_dev(d_t.data_ptr(), d_i.data_ptr(), d_w.data_ptr(), g_h.data_ptr(),
                                    g_n.data_ptr(), rows, hidden, EPS, stream()))
    assert np.array_equal(bits_of(g_h), oracle.embedding_f16(table, ids)), "gather is not bit-exact"
    u_h = torch.full((rows, hidden), float("nan"), dtype=torch.float16, device="cuda")
    u_n = torch.full((rows, hidden), float("nan"), dtype=torch.float16, device="cuda")
    ok(dev.vv_embedding_dev(d_t.data_ptr(), d_i.data_ptr(), u_h.data_ptr(), rows, hidden, stream()))
    ok(dev.vv_rmsnorm_dev(u_h.data_ptr(), d_w.data_ptr(), u_n.data_ptr(), rows, hidden, EPS, stream()))
    assert np.array_equal(bits_of(u_h), bits_of(g_h)) and np.array_equal(bits_of(u_n), bits_of(g_n))
    ref, rne = oracle.rmsnorm_f16(bits_of(g_h), w, EPS)
    assert_fp16_close(bits_of(g_n), ref, rne, f"gather+rmsnorm [{rows},{hidden}]")


# ── RoPE (config 3) ─────────────────────────────────────────────────────────

def rope_check(got_bits, x_bits, off, theta, what):
    ref, _ = oracle.rope_f16(x_bits, off, theta)
    return assert_rope_close(got_bits, x_bits, ref, what)


def test_rope_config3_prefill_q_and_k():
    T = 2048
    q = oracle.normal_f16((T, NQ, HD), 400)
    k = oracle.normal_f16((T, NK, HD), 401)
    d_q, d_k = to_dev(q), to_dev(k)
    ok(dev.vv_rope_dev(d_q.data_ptr(), T, NQ, HD, 0, None, 1e6, stream()))
    ok(dev.vv_rope_dev(d_k.data_ptr(), T, NK, HD, 0, None, 1e6, stream()))
    rope_check(bits_of(d_q), q, 0, 1e6, "rope Q")
    rope_check(bits_of(d_k), k, 0, 1e6, "rope K")
    # position 0 is the identity (cos 1, sin 0): bit-exact
    assert np.array_equal(bits_of(d_q)[0], q[0]) and np.array_equal(bits_of(d_k)[0], k[0])
    # one fused Q+K launch == the two single launches, bit for bit
    f_q, f_k = to_dev(q), to_dev(k)
    ok(dev.vv_rope_qk_dev(f_q.data_ptr(), f_k.data_ptr(), T, NQ, NK, HD, 0, None, 1e6, stream()))
    assert np.array_equal(bits_of(f_q), bits_of(d_q)) and np.array_equal(bits_of(f_k), bits_of(d_k))


@pytest.mark.parametrize("off", [8192, 913, 14448, 32767])
def test_rope_decode_scalar_and_device_position(off):
    """tests/test_decode_position.c:220-238: the position read from a device int
    must give exactly the bytes the scalar argument gives."""
    q = oracle.normal_f16((1, NQ, HD), 500 + off)
    a, b = to_dev(q), to_dev(q)
    d_pos = torch.tensor([off], dtype=torch.int32, device="cuda")
    ok(dev.vv_rope_dev(a.data_ptr(), 1, NQ, HD, off, None, 1e6, stream()))
    ok(dev.vv_rope_dev(b.data_ptr(), 1, NQ, HD, 0, d_pos.data_ptr(), 1e6, stream()))
    assert np.array_equal(bits_of(a), bits_of(b))
    assert not np.array_equal(bits_of(a), q)            # it actually rotated something
    rope_check(bits_of(a), q, off, 1e6, f"rope decode @{off}")


def test_rope_batched_equals_row_by_row_and_ragged_tail():
    T, off = 11, 5000                          # 11 rows: a ragged last workgroup
    q = oracle.normal_f16((T, NQ, HD), 600)
    k = oracle.normal_f16((T, NK, HD), 601)
    d_q, d_k = to_dev(q), to_dev(k)
    ok(dev.vv_rope_qk_dev(d_q.data_ptr(), d_k.data_ptr(), T, NQ, NK, HD, off, None, 1e6, stream()))
    rope_check(bits_of(d_q), q, off, 1e6, "rope ragged Q")
    rope_check(bits_of(d_k), k, off, 1e6, "rope ragged K")
    s_q = to_dev(q)
    for r in range(T):
        ok(dev.vv_rope_dev(s_q.data_ptr() + r * NQ * HD * 2, 1, NQ, HD, off + r, None, 1e6,
                           stream()))
    assert np.array_equal(bits_of(s_q), bits_of(d_q))


@pytest.mark.parametrize("heads,hd,theta,off", [(2, 128, 1e4, 0), (3, 64, 1e4, 77), (5, 256, 5e5, 1000),
                                                (1, 2, 1e4, 3), (7, 96, 1e6, 4000)])
def test_rope_other_shapes(heads, hd, theta, off):
    """theta 1e4 with 2 heads is tests/test_prefill_append.c:30,70; the rest
    exercise the generic kernel (head_dim != 128)."""
    T = 9
    x = oracle.normal_f16((T, heads, hd), 700 + hd)
    d_x = to_dev(x)
    ok(dev.vv_rope_dev(d_x.data_ptr(), T, heads, hd, off, None, theta, stream()))
    rope_check(bits_of(d_x), x, off, theta, f"rope heads={heads} hd={hd}")


def test_rope_unaligned_takes_generic_path_same_result():
    T, off = 6, 12345
    q = oracle.normal_f16((T, NQ, HD), 800)
    flat = torch.zeros(T * NQ * HD + 8, dtype=torch.float16, device="cuda")
    flat[1:1 + T * NQ * HD] = to_dev(q).reshape(-1)
    ok(dev.vv_rope_dev(flat.data_ptr() + 2, T, NQ, HD, off, None, 1e6, stream()))
    got = bits_of(flat)
    assert got[0] == 0 and not got[1 + T * NQ * HD:].any()
    d_q = to_dev(q)
    ok(dev.vv_rope_dev(d_q.data_ptr(), T, NQ, HD, off, None, 1e6, stream()))
    assert np.array_equal(got[1:1 + T * NQ * HD].reshape(T, NQ, HD), bits_of(d_q))


def test_bias_rope_equals_bias_add_then_rope():
    T, off = 37, 2048
    q = oracle.normal_f16((T, NQ, HD), 900)
    k = oracle.normal_f16((T, NK, HD), 901)
    qb = oracle.normal_f16((NQ * HD,), 902, std=0.5)
    kb = oracle.normal_f16((NK * HD,), 903, std=0.5)
    a_q, a_k, d_qb, d_kb = to_dev(q), to_dev(k), to_dev(qb), to_dev(kb)
    ok(dev.vv_bias_add_dev(a_q.data_ptr(), d_qb.data_ptr(), T, NQ * HD, stream()))
    ok(dev.vv_bias_add_dev(a_k.data_ptr(), d_kb.data_ptr(), T, NK * HD, stream()))
    assert np.array_equal(bits_of(a_q).reshape(T, -1), oracle.bias_add_f16(q.reshape(T, -1), qb))
    assert np.array_equal(bits_of(a_k).reshape(T, -1), oracle.bias_add_f16(k.reshape(T, -1), kb))
    ok(dev.vv_rope_qk_dev(a_q.data_ptr(), a_k.data_ptr(), T, NQ, NK, HD, off, None, 1e6, stream()))
    f_q, f_k = to_dev(q), to_dev(k)
    ok(dev.vv_bias_rope_qk_dev(f_q.data_ptr(), f_k.data_ptr(), d_qb.data_ptr(), d_kb.data_ptr(),
                               T, NQ, NK, HD, off, None, 1e6, stream()))
    assert np.array_equal(bits_of(f_q), bits_of(a_q)) and np.array_equal(bits_of(f_k), bits_of(a_k))
    biased_q = oracle.bias_add_f16(q.reshape(T, -1), qb).reshape(T, NQ, HD)
    rope_check(bits_of(f_q), biased_q, off, 1e6, "bias+rope Q")


@pytest.mark.parametrize("T,off", [(1000, 0), (3001, 8192), (770, 31000)])
def test_rope_mid_size_launches_agree_with_short_ones(T, off):
    """A thousand to a few thousand positions run one wave per position, other lengths a
    workgroup per position: same angle, same sincosf, same rotation, so the same bits - checked
    against one-row launches, the device-side position and the bias form, then the oracle."""
    q = oracle.normal_f16((T, NQ, HD), 950 + T)
    k = oracle.normal_f16((T, NK, HD), 951 + T)
    d_q, d_k = to_dev(q), to_dev(k)
    ok(dev.vv_rope_qk_dev(d_q.data_ptr(), d_k.data_ptr(), T, NQ, NK, HD, off, None, 1e6, stream()))
    rope_check(bits_of(d_q), q, off, 1e6, f"rope Q T={T}")
    rope_check(bits_of(d_k), k, off, 1e6, f"rope K T={T}")
    for r in (0, 1, T // 2, T - 1):
        one_q, one_k = to_dev(q[r:r + 1]), to_dev(k[r:r + 1])
        ok(dev.vv_rope_qk_dev(one_q.data_ptr(), one_k.data_ptr(), 1, NQ, NK, HD, off + r, None, 1e6, stream()))
        assert np.array_equal(bits_of(one_q)[0], bits_of(d_q)[r]) and np.array_equal(bits_of(one_k)[0], bits_of(d_k)[r])
    p_q, p_k = to_dev(q), to_dev(k)
    d_pos = torch.tensor([off], dtype=torch.int32, device="cuda")
    ok(dev.vv_rope_qk_dev(p_q.data_ptr(), p_k.data_ptr(), T, NQ, NK, HD, 0, d_pos.data_ptr(), 1e6, stream()))
    assert np.array_equal(bits_of(p_q), bits_of(d_q)) and np.array_equal(bits_of(p_k), bits_of(d_k))
    s_k = to_dev(k)                                  # K alone: 4 heads, a short launch in workgroup form
    ok(dev.vv_rope_dev(s_k.data_ptr(), T, NK, HD, off, None, 1e6, stream()))
    assert np.array_equal(bits_of(s_k), bits_of(d_k))
    qb = oracle.normal_f16((NQ * HD,), 952, std=0.5)
    kb = oracle.normal_f16((NK * HD,), 953, std=0.5)
    a_q, a_k, d_qb, d_kb = to_dev(q), to_dev(k), to_dev(qb), to_dev(kb)
    ok(dev.vv_bias_add_dev(a_q.data_ptr(), d_qb.data_ptr(), T, NQ * HD, stream()))
    ok(dev.vv_bias_add_dev(a_k.data_ptr(), d_kb.data_ptr(), T, NK * HD, stream()))
    ok(dev.vv_rope_qk_dev(a_q.data_ptr(), a_k.data_ptr(), T, NQ, NK, HD, off, None, 1e6, stream()))
    f_q, f_k = to_dev(q), to_dev(k)
    ok(dev.vv_bias_rope_qk_dev(f_q.data_ptr(), f_k.data_ptr(), d_qb.data_ptr(), None, T, NQ, NK, HD, off, None,
                               1e6, stream()))
    assert np.array_equal(bits_of(f_q), bits_of(a_q)) and np.array_equal(bits_of(f_k), bits_of(d_k))
    f_q, f_k = to_dev(q), to_dev(k)
    ok(dev.vv_bias_rope_qk_dev(f_q.data_ptr(), f_k.data_ptr(), d_qb.data_ptr(), d_kb.data_ptr(), T, NQ, NK, HD,
                               off, None, 1e6, stream()))
    assert np.array_equal(bits_of(f_q), bits_of(a_q)) and np.array_equal(bits_of(f_k), bits_of(a_k))


# ── SwiGLU (config 4) ───────────────────────────────────────────────────────

@pytest.mark.parametrize("rows", [1, 4096])
def test_swiglu_config4(rows):
    g = oracle.normal_f16((rows, I_FF), 1000 + rows, std=2.0)
    u = oracle.normal_f16((rows, I_FF), 2000 + rows, std=2.0)
    ref, rne = oracle.swiglu_f16(g, u)
    d_g, d_u = to_dev(g), to_dev(u)
    d_o = torch.empty_like(d_g)
    ok(dev.vv_swiglu_dev(d_g.data_ptr(), d_u.data_ptr(), d_o.data_ptr(), rows * I_FF, stream()))
    assert_fp16_close(bits_of(d_o), ref, rne, f"swiglu T={rows}", max_mismatch=0.005)
    # in place over gate, the way the decoder calls it (decoder.c:977): same bits
    ok(dev.vv_swiglu_dev(d_g.data_ptr(), d_u.data_ptr(), d_g.data_ptr(), rows * I_FF, stream()))
    assert np.array_equal(bits_of(d_g), bits_of(d_o))
    assert np.array_equal(bits_of(d_u), u)


def test_swiglu_special_values_odd_length_unaligned():
    n = 100_003                                   # odd: the reference's scalar kernel case
    g = oracle.normal_f16((n,), 31, std=4.0)
    u = oracle.normal_f16((n,), 32, std=1.0)
    sp = oracle.narrow(np.array([0.0, -0.0, 65504.0, -65504.0, 88.0, -88.0, 11.0, -11.0,
                                 6e-8, -6e-8, 1.0, -1.0, 20.0, -20.0], np.float32))
    g[:sp.size] = sp
    u[:4] = oracle.narrow(np.array([5.0, 5.0, 2.0, 2.0], np.float32))
    u[20:24] = oracle.narrow(np.array([0.0, -0.0, 65504.0, -65504.0], np.float32))
    with np.errstate(over="ignore"):
        ref, rne = oracle.swiglu_f16(g, u)
    d_g, d_u = to_dev(g), to_dev(u)
    d_o = torch.empty_like(d_g)
    ok(dev.vv_swiglu_dev(d_g.data_ptr(), d_u.data_ptr(), d_o.data_ptr(), n, stream()))
    got = bits_of(d_o)
    assert not np.isnan(oracle.widen(got)).any()
    assert got[0] == rne[0] and got[1] == rne[1] and got[3] == rne[3]   # signed zeros
    assert got[2] == 0x7C00                                             # 2 * 65504 overflows FP16
    assert_fp16_close(got, ref, rne, "swiglu specials", max_mismatch=0.005)
    flat = torch.zeros(n + 8, dtype=torch.float16, device="cuda")
    ok(dev.vv_swiglu_dev(d_g.data_ptr(), d_u.data_ptr(), flat.data_ptr() + 2, n, stream()))
    got2 = bits_of(flat)
    assert got2[0] == 0 and not got2[1 + n:].any()
    assert np.array_equal(got2[1:1 + n], got)


@pytest.mark.parametrize("rows,inter", [(5, 18944), (3, 1000), (2, 37)])
def test_swiglu_fused_layout(rows, inter):
    gu = oracle.normal_f16((rows, 2 * inter), 40 + inter, std=2.0)
    ref, rne = oracle.swiglu_fused_f16(gu)
    d_gu = to_dev(gu)
    d_o = torch.empty(rows, inter, dtype=torch.float16, device="cuda")
    ok(dev.vv_swiglu_fused_dev(d_gu.data_ptr(), d_o.data_ptr(), rows, inter, stream()))
    assert_fp16_close(bits_of(d_o), ref, rne, f"swiglu_fused [{rows},{inter}]", max_mismatch=0.005)
    # == the two-pointer form on the same values
    g = np.ascontiguousarray(gu[:, :inter])
    u = np.ascontiguousarray(gu[:, inter:])
    d_g, d_u = to_dev(g), to_dev(u)
    d_o2 = torch.empty_like(d_o)
    ok(dev.vv_swiglu_dev(d_g.data_ptr(), d_u.data_ptr(), d_o2.data_ptr(), rows * inter, stream()))
    assert np.array_equal(bits_of(d_o), bits_of(d_o2))


# ── embedding gather and the first-layer chain (config 5) ───────────────────

@pytest.fixture(scope="module")
def qwen_table():
    """[152064, 3584] FP16 ~N(0, 0.02), made on the device (1.09 GB) and read
    back once so the oracle sees the same bytes."""
    gen = torch.Generator(device="cuda").manual_seed(5)
    t = (torch.randn(V, H, generator=gen, device="cuda", dtype=torch.float32) * 0.02).half()
    return t, bits_of(t)


def test_embedding_config5_bit_exact_and_chain(qwen_table):
    d_table, table = qwen_table
    T = 14449
    ids = oracle.ids(T, 5, V)
    ids[:4] = [0, V - 1, V - 1, 0]                       # first, last, duplicates
    d_ids = torch.from_numpy(ids).cuda()
    d_out = torch.zeros(T, H, dtype=torch.float16, device="cuda")
    ok(dev.vv_embedding_dev(d_table.data_ptr(), d_ids.data_ptr(), d_out.data_ptr(), T, H, stream()))
    want = oracle.embedding_f16(table, ids)
    assert np.array_equal(bits_of(d_out), want), "gather must be bit-exact"

    w = weight(H)
    d_w = to_dev(w)
    d_n = torch.empty_like(d_out)
    ok(dev.vv_rmsnorm_dev(d_out.data_ptr(), d_w.data_ptr(), d_n.data_ptr(), T, H, EPS, stream()))
    ref, rne = oracle.rmsnorm_f16(want, w, EPS)
    assert_fp16_close(bits_of(d_n), ref, rne, "gather -> rmsnorm")

    # fused gather+norm == the two calls, bit for bit
    f_h = torch.zeros_like(d_out)
    f_n = torch.zeros_like(d_out)
    ok(dev.vv_embedding_rmsnorm_dev(d_table.data_ptr(), d_ids.data_ptr(), d_w.data_ptr(),
                                    f_h.data_ptr(), f_n.data_ptr(), T, H, EPS, stream()))
    assert np.array_equal(bits_of(f_h), want)
    assert np.array_equal(bits_of(f_n), bits_of(d_n))


def test_embedding_any_bit_pattern_other_widths_and_decode_row():
    rng = np.random.default_rng(12)
    for hidden, vocab, T in [(3584, 300, 1), (100, 50, 33), (4096, 64, 17), (8960, 20, 5), (1, 10, 10)]:
        table = rng.integers(0, 65536, size=(vocab, hidden), dtype=np.uint16)   # NaNs, infs, subnormals
        ids = oracle.ids(T, hidden, vocab)
        d_t, d_i = to_dev(table), torch.from_numpy(ids).cuda()
        d_o = torch.zeros(T, hidden, dtype=torch.float16, device="cuda")
        ok(dev.vv_embedding_dev(d_t.data_ptr(), d_i.data_ptr(), d_o.data_ptr(), T, hidden, stream()))
        assert np.array_equal(bits_of(d_o), table[ids]), (hidden, vocab, T)


# ── bias add and conversions ─────────────────────────────────────────────────

@pytest.mark.parametrize("M,N", [(285, 3584), (7, 512), (3, 100), (1, 18944)])
def test_bias_add_bit_exact(M, N):
    x = oracle.normal_f16((M, N), 50 + N, std=3.0)
    b = oracle.normal_f16((N,), 51, std=1.0)
    d_x, d_b = to_dev(x), to_dev(b)
    ok(dev.vv_bias_add_dev(d_x.data_ptr(), d_b.data_ptr(), M, N, stream()))
    assert np.array_equal(bits_of(d_x), oracle.bias_add_f16(x, b))


def test_fp16_fp32_conversions_bit_exact():
    h = np.arange(65536, dtype=np.uint16)
    d_h = to_dev(h)
    d_f = torch.empty(65536, dtype=torch.float32, device="cuda")
    ok(dev.vv_fp16_to_fp32_dev(d_h.data_ptr(), d_f.data_ptr(), 65536, stream()))
    got = d_f.cpu().numpy()
    want = oracle.widen(h)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.isnan(got[nan]).all()
    f = oracle.normal_f32((500_001,), 60, std=50.0)
    f[:5] = [65504.0, 65520.0, 1e-8, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11]
    d_in = torch.from_numpy(f).cuda()
    d_out = torch.empty(f.size, dtype=torch.float16, device="cuda")
    ok(dev.vv_fp32_to_fp16_dev(d_in.data_ptr(), d_out.data_ptr(), f.size, stream()))
    assert np.array_equal(bits_of(d_out), oracle.narrow(f))


# ── full prefill size (T = 14449): size-independent properties ──────────────

def test_full_size_properties_T14449():
    """At the benchmark's full size the oracle is run on sampled rows only; the rest
    is covered by equalities that hold at any size."""
    T = 14449
    gen = torch.Generator(device="cuda").manual_seed(14449)
    res = torch.randn(T, H, generator=gen, device="cuda").half()
    x = torch.randn(T, H, generator=gen, device="cuda").half()
    w = weight(H)
    d_w = to_dev(w)
    # fused add+norm == add then norm (bit-exact), everywhere
    f_res, f_n = res.clone(), torch.empty_like(res)
    ok(dev.vv_add_rmsnorm_dev(f_res.data_ptr(), x.data_ptr(), d_w.data_ptr(), f_n.data_ptr(),
                              T, H, EPS, stream()))
    u_res, u_n = res.clone(), torch.empty_like(res)
    ok(dev.vv_residual_add_dev(u_res.data_ptr(), x.data_ptr(), T * H, stream()))
    ok(dev.vv_rmsnorm_dev(u_res.data_ptr(), d_w.data_ptr(), u_n.data_ptr(), T, H, EPS, stream()))
    torch.cuda.synchronize()
    assert torch.equal(f_res, u_res) and torch.equal(f_n, u_n)
    # sampled rows (first, last, around workgroup boundaries) against the oracle
    rows = np.array([0, 1, 2, 3, 4, 5, 4095, 4096, 8191, 14444, 14445, 14446, 14447, 14448])
    rb, xb = bits_of(res)[rows], bits_of(x)[rows]
    want_res, nref, nrne = oracle.add_rmsnorm_f16(np.ascontiguousarray(rb), np.ascontiguousarray(xb),
                                                  w, EPS)
    assert np.array_equal(bits_of(f_res)[rows], want_res)
    assert_fp16_close(bits_of(f_n)[rows], nref, nrne, "add+rmsnorm sampled rows")
    del f_res, f_n, u_res, u_n, res, x

    # SwiGLU: in place == out of place on all 273.7M elements; slices against the oracle
    n = T * I_FF
    g = (torch.randn(n, generator=gen, device="cuda") * 2).half()
    u = (torch.randn(n, generator=gen, device="cuda") * 2).half()
    o = torch.empty_like(g)
    ok(dev.vv_swiglu_dev(g.data_ptr(), u.data_ptr(), o.data_ptr(), n, stream()))
    for lo in (0, n // 2 - 12345, n - 1_000_000):
        ref, rne = oracle.swiglu_f16(bits_of(g[lo:lo + 1_000_000]), bits_of(u[lo:lo + 1_000_000]))
        assert_fp16_close(bits_of(o[lo:lo + 1_000_000]), ref, rne, f"swiglu slice @{lo}",
                          max_mismatch=0.005)
    ok(dev.vv_swiglu_dev(g.data_ptr(), u.data_ptr(), g.data_ptr(), n, stream()))
    torch.cuda.synchronize()
    assert torch.equal(g, o)
    del g, u, o

    # RoPE at the last positions of the prompt, Q and K in one launch
    q = torch.randn(T, NQ, HD, generator=gen, device="cuda").half()
    k = torch.randn(T, NK, HD, generator=gen, device="cuda").half()
    q0, k0 = bits_of(q), bits_of(k)
    ok(dev.vv_rope_qk_dev(q.data_ptr(), k.data_ptr(), T, NQ, NK, HD, 0, None, 1e6, stream()))
    lo = T - 64
    rope_check(bits_of(q)[lo:], np.ascontiguousarray(q0[lo:]), lo, 1e6, "rope Q tail rows")
    rope_check(bits_of(k)[lo:], np.ascontiguousarray(k0[lo:]), lo, 1e6, "rope K tail rows")
    # per-pair norms are preserved everywhere (a rotation), up to FP16 rounding
    qf, q0f = q.float(), torch.from_numpy(q0.view(np.float16)).cuda().float()
    n_after = qf[..., :64] ** 2 + qf[..., 64:] ** 2
    n_before = q0f[..., :64] ** 2 + q0f[..., 64:] ** 2
    assert torch.allclose(n_after, n_before, rtol=4e-3, atol=1e-4)
