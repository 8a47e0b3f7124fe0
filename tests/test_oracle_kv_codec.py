"""The oracle's FP8 KV-cache codec, pinned by what the two formats fix.

The reference holds this codec only as accelerator code (src/cuda/kv_codec.cuh),
so there is no compiled CPU form to compare with. Instead: every one of the
256 codes must decode to the closed-form value of its fields, and every FP16
input (all 65536 of them: the cache is written from FP16) must encode to a
representable value nearest to it, ties resolved as the format's rounding
says, with the documented handling of zero, NaN and out-of-range inputs.
"""
import numpy as np
import pytest

import oracle

FORMATS = {"e4m3": dict(e5m2=False, mant=3, bias=7, max_code=0x7E), "e5m2": dict(e5m2=True, mant=2, bias=15, max_code=0x7B)}


def closed_form(code, mant, bias):
    e, m = (code >> mant) & ((1 << (7 - mant)) - 1), code & ((1 << mant) - 1)
    mag = m * 2.0 ** (1 - bias - mant) if e == 0 else (1 + m / 2 ** mant) * 2.0 ** (e - bias)
    return -mag if code & 0x80 else mag


@pytest.mark.parametrize("name", FORMATS)
def test_every_code_decodes_to_its_closed_form(name):
    f = FORMATS[name]
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.fp8_decode(codes, f["e5m2"]).astype(np.float64)
    want = np.array([closed_form(int(c), f["mant"], f["bias"]) for c in codes])
    assert np.array_equal(got, want)
    assert np.array_equal(np.signbit(got), (codes & 0x80) != 0)


@pytest.mark.parametrize("name", FORMATS)
def test_every_fp16_input_encodes_to_a_nearest_value(name):
    f = FORMATS[name]
    bits = np.arange(65536, dtype=np.uint16)
    x = oracle.widen(bits)
    codes = oracle.fp8_encode(x, f["e5m2"])
    finite = np.isfinite(x)
    # zero and NaN: a signed zero
    assert np.array_equal(codes[(x == 0) | np.isnan(x)] & 0x7F, np.zeros(((x == 0) | np.isnan(x)).sum(), np.uint8))
    assert np.array_equal(codes & 0x80, ((bits >> 8) & 0x80).astype(np.uint8))
    # never beyond the largest finite code
    assert (codes & 0x7F).max() == f["max_code"]
    # nearest: no representable magnitude up to the largest finite one is closer
    table = np.array([closed_form(c, f["mant"], f["bias"]) for c in range(f["max_code"] + 1)])
    a = np.abs(x[finite]).astype(np.float64)
    got = np.abs(oracle.fp8_decode(codes[finite], f["e5m2"]).astype(np.float64))
    best = np.abs(a[:, None] - table[None, :]).min(axis=1)
    assert np.array_equal(np.abs(a - got), best)
    # ties between two normals go to the even mantissa; infinities saturate
    inf_codes = codes[np.isinf(x)] & 0x7F
    assert (inf_codes == f["max_code"]).all()
    idx = np.abs(a[:, None] - table[None, :]).argsort(axis=1)[:, :2]
    d0 = np.abs(a - table[idx[:, 0]])
    d1 = np.abs(a - table[idx[:, 1]])
    tie = (d0 == d1) & (a < table[-1])
    lo = np.minimum(idx[tie, 0], idx[tie, 1])
    normal_tie = lo >= (1 << f["mant"])                       # both neighbours are normals
    chosen = (codes[finite][tie] & 0x7F).astype(np.int64)
    assert ((chosen[normal_tie] & 1) == 0).all()


def test_reference_key_and_store():
    rng = np.random.default_rng(0)
    k = oracle.normal_f16((37, 4, 128), 1, mean=3.0, std=2.0)
    ref = oracle.kv_build_ref(k)
    mean = oracle.widen(k).astype(np.float64).mean(axis=0)
    assert np.max(np.abs(oracle.widen(ref) - mean)) <= np.max(np.abs(mean)) * 2.0 ** -10
    for e5m2 in (False, True):
        store = oracle.kv_store_fp8(k, ref, e5m2)
        want = oracle.fp8_encode(oracle.widen(k) - oracle.widen(ref)[None], e5m2)
        assert np.array_equal(store, want)
        assert np.array_equal(oracle.kv_store_fp8(k, None, e5m2), oracle.fp8_encode(oracle.widen(k), e5m2))


# ── TurboQuant ──────────────────────────────────────────────────────────────
TQ = {3: dict(bits=4, snr_db=20.2), 4: dict(bits=3, snr_db=14.6), 5: dict(bits=2, snr_db=9.3), 6: dict(bits=1.5, snr_db=7.0)}


def test_rotation_is_the_scaled_hadamard_matrix_times_signs():
    """Against the explicit 128 x 128 matrix H[i][j] = (-1)^popcount(i & j) / sqrt(128)
    in FP64: rotate(x) = H (s * x) for ONE +-1 diagonal s (read off by rotating
    nothing but its inverse), the inverse undoes it, and norms are kept."""
    idx = np.arange(128)
    H = np.array([[(-1.0) ** bin(i & j).count("1") for j in idx] for i in idx]) / np.sqrt(128.0)
    x = oracle.normal_f16((40, 128), 1, std=2.0)
    xf = oracle.widen(x).astype(np.float64)
    y = oracle.widen(oracle.kv_rotate(x)).astype(np.float64)
    # the sign diagonal: rotate a vector of ones, undo the Hadamard part
    ones = oracle.narrow(np.ones((1, 128), np.float32))
    s = np.rint(H.T @ oracle.widen(oracle.kv_rotate(ones)).astype(np.float64)[0] * 1.0)
    s = np.sign(H @ oracle.widen(oracle.kv_rotate(ones)).astype(np.float64)[0])
    assert set(np.unique(s)) <= {-1.0, 1.0} and 20 < (s < 0).sum() < 108
    want = (xf * s[None]) @ H.T
    assert np.max(np.abs(y - want)) <= 2.0 ** -10 * np.max(np.abs(want)) + 1e-6
    back = oracle.widen(oracle.kv_rotate(oracle.kv_rotate(x), inverse=True)).astype(np.float64)
    assert np.max(np.abs(back - xf)) <= 3 * 2.0 ** -10 * np.max(np.abs(xf))
    assert np.allclose((y ** 2).sum(1), (xf ** 2).sum(1), rtol=3e-3)


def gaussian_cell_means(levels):
    """Centroids of N(0,1) over the cells bounded by the mid-points of `levels`."""
    from scipy.stats import norm
    edges = np.concatenate([[-np.inf], (levels[1:] + levels[:-1]) / 2, [np.inf]])
    lo, hi = edges[:-1], edges[1:]
    return (norm.pdf(lo) - norm.pdf(hi)) / (norm.cdf(hi) - norm.cdf(lo))


@pytest.mark.parametrize("fmt", [3, 4, 5])
def test_scalar_levels_are_the_lloyd_max_fixed_point(fmt):
    """Store a vector whose RMS is 1 and read the levels back through the codec;
    each must be the mean of a unit Gaussian over its own cell."""
    nb = TQ[fmt]["bits"]
    # every code value appears when the stored values are the cell centres; read the table off the dequantiser
    store = np.zeros((1, 1, oracle.kv_bytes_per_vec(fmt)), np.uint8)
    n_levels = 1 << nb
    codes = np.arange(128) % n_levels
    stream = 0
    for d, c in enumerate(codes):
        stream |= int(c) << (d * nb)
    store[0, 0] = np.frombuffer(stream.to_bytes(oracle.kv_bytes_per_vec(fmt), "little"), np.uint8)
    one = oracle.narrow(np.ones((1, 1), np.float32))
    levels = oracle.widen(oracle.kv_unpack(store, one, fmt))[0, 0, :n_levels].astype(np.float64)
    assert np.all(np.diff(levels) > 0) and np.allclose(levels, -levels[::-1], atol=1e-3)
    assert np.max(np.abs(levels - gaussian_cell_means(levels))) < 4e-3        # FP16 read-back of 6-digit tables


@pytest.mark.parametrize("fmt", [3, 4, 5, 6])
def test_codes_are_nearest_and_reach_the_quoted_signal_to_noise(fmt):
    """On Gaussian vectors: unpack(store(x)) is, per value (per pair for 1.5
    bits), the nearest entry of the scaled table, and the signal-to-noise ratio
    is the one the reference quotes for the format (kv_codec.cuh:40-41)."""
    n = 64
    x = oracle.normal_f16((n, 1, 128), 7 + fmt, std=1.7)
    store, meta = oracle.kv_store_tq(x, None, fmt)
    assert store.shape[-1] == oracle.kv_bytes_per_vec(fmt)
    y = oracle.widen(oracle.kv_rotate(x)).astype(np.float64)[:, 0]              # what was quantised (to FP16 rounding)
    got = oracle.widen(oracle.kv_unpack(store, meta, fmt)).astype(np.float64)[:, 0]
    sigma = oracle.widen(meta).astype(np.float64)[:, 0]
    assert np.allclose(sigma, np.sqrt((y ** 2).mean(1)), rtol=2e-3)
    err = ((got - y) ** 2).sum() / (y ** 2).sum()
    snr = -10 * np.log10(err)
    assert abs(snr - TQ[fmt]["snr_db"]) < 0.5, snr
    # nearest: no other table entry is closer (up to the FP16 rounding of the rotated input)
    if fmt != 6:
        vals = np.sort((got / sigma[:, None]).ravel())
        table = np.array([c.mean() for c in np.split(vals, np.nonzero(np.diff(vals) > 0.05)[0] + 1)])
        assert len(table) == 1 << TQ[fmt]["bits"]
        d_best = np.abs(y[:, :, None] / sigma[:, None, None] - table[None, None, :]).min(-1)
        d_got = np.abs(y / sigma[:, None] - got / sigma[:, None])
        assert np.max(d_got - d_best) < 5e-3
    else:
        pairs = (got / sigma[:, None]).reshape(n, 64, 2)
        flat = pairs.reshape(-1, 2)
        table = []
        for p in flat:                                   # cluster the read-back pairs (FP16 noise apart)
            if not any(np.abs(p - t).max() < 0.05 for t in table):
                table.append(p)
        table = np.array(table)
        assert len(table) == 8
        yp = (y / sigma[:, None]).reshape(n, 64, 2)
        d_best = ((yp[:, :, None, :] - table[None, None]) ** 2).sum(-1).min(-1)
        d_got = ((yp - pairs) ** 2).sum(-1)
        assert np.max(d_got - d_best) < 1e-2


def test_turboquant_reference_key_and_fp8_dequant_agree_with_the_codec():
    k = oracle.normal_f16((9, 4, 128), 3, mean=2.0, std=1.0)
    ref = oracle.kv_build_ref(k)
    centred = oracle.narrow(oracle.widen(k) - oracle.widen(ref)[None])
    for fmt in (3, 6):
        a, ma = oracle.kv_store_tq(k, ref, fmt)
        # subtracting in FP32 before the transform is not subtracting FP16-rounded differences, but nearly
        b, mb = oracle.kv_store_tq(centred, None, fmt)
        assert (a != b).mean() < 0.02 and np.abs(oracle.widen(ma) - oracle.widen(mb)).max() < 1e-2
    for fmt, e5m2 in ((1, False), (2, True)):
        codes = oracle.kv_store_fp8(k, None, e5m2)
        assert np.array_equal(oracle.widen(oracle.kv_dequant(codes, None, None, fmt)), oracle.fp8_decode(codes, e5m2))
        assert np.array_equal(oracle.kv_dequant(codes, None, None, fmt), oracle.kv_unpack(codes, None, fmt))


@pytest.mark.parametrize("fmt", [3, 4, 5, 6])
def test_dequant_returns_to_the_original_space(fmt):
    """The seam's dequantiser undoes the rotation and adds the reference key back
    (kv_quant.cu:325-334): it is the inverse transform of the unpacked vector to
    FP16 rounding, and, the transform being orthogonal, lands as close to the
    original vector as the unpacked one is to the rotated one."""
    k = oracle.normal_f16((33, 4, 128), 21, mean=1.5, std=1.0)
    ref = oracle.kv_build_ref(k)
    store, meta = oracle.kv_store_tq(k, ref, fmt)
    plain = oracle.widen(oracle.kv_dequant(store, meta, None, fmt)).astype(np.float64)
    by_hand = oracle.widen(oracle.kv_rotate(oracle.kv_unpack(store, meta, fmt), inverse=True)).astype(np.float64)
    assert np.max(np.abs(plain - by_hand)) < 6e-3                 # one rounding against two
    with_ref = oracle.widen(oracle.kv_dequant(store, meta, ref, fmt)).astype(np.float64)
    assert np.max(np.abs(with_ref - (plain + oracle.widen(ref)[None]))) < 6e-3
    x = oracle.widen(k).astype(np.float64)
    centred = x - oracle.widen(ref)[None]
    err_orig = ((with_ref - x) ** 2).sum() / (centred ** 2).sum()
    y = oracle.widen(oracle.kv_rotate(oracle.narrow(centred.astype(np.float32)))).astype(np.float64)
    err_rot = ((oracle.widen(oracle.kv_unpack(store, meta, fmt)) - y) ** 2).sum() / (y ** 2).sum()
    assert abs(-10 * np.log10(err_orig) - TQ[fmt]["snr_db"]) < 0.6
    assert abs(err_orig - err_rot) < 0.05 * err_rot
