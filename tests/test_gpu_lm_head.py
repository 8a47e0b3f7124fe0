"""GPU parity tests of the LM head (FP16 table x FP16 vector -> FP32 logits) and
the on-device greedy argmax, through the C ABI.

Logits: FP32 accumulation over K against the oracle's double-accumulated
product; bar 1e-5 of max|logit| (the FP32 bar) and elementwise 2e-6 of
sum|x||w|. Argmax: the token the oracle's in-order scan picks from the DEVICE's
logits, exactly, including ties (lowest index), all-negative vectors, -inf and
NaN entries, and vocabulary sizes that are not a multiple of anything.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, ok, stream, to_dev
from conftest import scaled_rel_err

pytestmark = pytest.mark.gpu


def argmax(d_logits, V):
    sv = torch.empty(256, dtype=torch.float32, device="cuda")
    si = torch.empty(256, dtype=torch.int32, device="cuda")
    tok = torch.full((1,), -7, dtype=torch.int32, device="cuda")
    val = torch.zeros(1, dtype=torch.float32, device="cuda")
    ok(dev.vv_argmax_dev(d_logits.data_ptr(), V, sv.data_ptr(), si.data_ptr(), tok.data_ptr(), val.data_ptr(),
                         stream()))
    tok2 = torch.full((1,), -7, dtype=torch.int32, device="cuda")
    ok(dev.vv_argmax_dev(d_logits.data_ptr(), V, sv.data_ptr(), si.data_ptr(), tok2.data_ptr(), None, stream()))
    torch.cuda.synchronize()
    assert int(tok2.item()) == int(tok.item())
    return int(tok.item()), float(val.item())


@pytest.mark.parametrize("V,K", [(152064, 3584), (1000, 1536), (77, 264), (5, 8), (300, 100)])
def test_lm_head_logits_and_token(V, K):
    x = oracle.normal_f16((1, K), V + K)
    w = oracle.normal_f16((V, K), 2 * V + 1, std=K ** -0.5)
    d_x, d_w = to_dev(x), to_dev(w)
    logits = torch.full((V,), float("nan"), dtype=torch.float32, device="cuda")
    ok(dev.vv_lm_head_gemv_dev(d_x.data_ptr(), d_w.data_ptr(), logits.data_ptr(), V, K, stream()))
    torch.cuda.synchronize()
    got = logits.cpu().numpy()
    ref = oracle.gemm_f16w(oracle.widen(x), w)[0].astype(np.float64)
    assert scaled_rel_err(got, ref) <= 1e-5
    mag = np.abs(oracle.widen(w)).astype(np.float64) @ np.abs(oracle.widen(x[0])).astype(np.float64)
    assert np.max(np.abs(got - ref) / (2e-6 * mag + 1e-30)) <= 1.0
    tok, val = argmax(logits, V)
    want_tok, want_val = oracle.argmax_first(got)
    assert (tok, val) == (want_tok, want_val)


@pytest.mark.parametrize("V", [1, 2, 255, 256, 257, 65536, 65537, 152064])
def test_argmax_ties_and_odd_sizes(V):
    rng = np.random.default_rng(V)
    x = rng.standard_normal(V).astype(np.float32)
    cases = [x, -np.abs(x) - 1.0]                                     # all negative
    tied = x.copy()
    hits = rng.choice(V, size=min(V, 5), replace=False)
    tied[hits] = 9.5                                                   # several equal maxima: the lowest index wins
    cases.append(tied)
    if V > 4:
        odd = x.copy()
        odd[::3] = -np.inf
        odd[1], odd[V // 2] = np.nan, np.nan                           # a NaN never wins
        cases.append(odd)
    for c in cases:
        tok, val = argmax(torch.from_numpy(c).cuda(), V)
        finite_first = np.where(np.isnan(c), -np.inf, c)
        assert tok == int(np.argmax(finite_first)), (V, tok)
        assert val == float(finite_first.max())


def test_lm_head_edges():
    d = torch.ones(64, dtype=torch.float16, device="cuda")
    f = torch.zeros(64, dtype=torch.float32, device="cuda")
    p = d.data_ptr()
    assert dev.vv_lm_head_gemv_dev(None, p, f.data_ptr(), 4, 8, stream()) == dev.VV_ERR_NULL_PTR
    assert dev.vv_lm_head_gemv_dev(p, p, f.data_ptr(), 0, 8, stream()) == dev.VV_OK
    assert dev.vv_argmax_dev(f.data_ptr(), 4, None, f.data_ptr(), f.data_ptr(), None, stream()) == dev.VV_ERR_NULL_PTR
    # an unaligned vector takes the 2-byte kernel
    ok(dev.vv_lm_head_gemv_dev(p + 2, p + 32, f.data_ptr(), 3, 12, stream()))
    torch.cuda.synchronize()
    assert f[:3].tolist() == [12.0, 12.0, 12.0]
