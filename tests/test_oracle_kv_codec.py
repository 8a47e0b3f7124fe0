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
