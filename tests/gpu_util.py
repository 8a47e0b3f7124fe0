"""Helpers for the GPU parity tests: device buffers from FP16 bit patterns,
read-back as bit patterns, and the two acceptance bars.

The HIP library is reached only through its C ABI (ctypes); torch is used for
device memory and the current stream, nothing else.
"""
import numpy as np
import torch

import oracle
from conftest import scaled_rel_err, ulp16_diff
from __graft_entry__ import load_device

dev = load_device()

FP16_TOL = 2e-3      # the acceptance bar for FP16 outputs: max|err| / max|ref|


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def to_dev(bits: np.ndarray) -> torch.Tensor:
    """uint16 FP16 bit patterns -> device float16 tensor of the same shape."""
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.float16)).cuda()


def bits_of(t: torch.Tensor) -> np.ndarray:
    torch.cuda.synchronize()
    return t.detach().cpu().contiguous().numpy().view(np.uint16)


def ok(status: int) -> None:
    assert status == dev.VV_OK, f"status {status}"


def assert_fp16_close(got_bits, ref_f32, rne_bits, what, max_ulp=1, max_mismatch=0.02):
    """The stated bar (scaled error <= 2e-3) plus a much tighter one of our
    own: no element more than `max_ulp` FP16 steps from the correctly rounded
    oracle value, and only a small fraction off at all."""
    got_bits, rne_bits = np.asarray(got_bits).reshape(-1), np.asarray(rne_bits).reshape(-1)
    ref_f32 = np.asarray(ref_f32).reshape(-1)
    # where the correctly rounded answer is inf or NaN the device must say the same
    finite = (rne_bits & 0x7C00) != 0x7C00
    odd_got, odd_want = got_bits[~finite], rne_bits[~finite]
    is_nan = (odd_want & 0x3FF) != 0
    assert np.array_equal(odd_got[~is_nan], odd_want[~is_nan]), f"{what}: infinities differ"
    assert (((odd_got[is_nan] & 0x7C00) == 0x7C00) & ((odd_got[is_nan] & 0x3FF) != 0)).all(), \
        f"{what}: NaN expected"
    got_bits, rne_bits, ref_f32 = got_bits[finite], rne_bits[finite], ref_f32[finite]
    got = oracle.widen(got_bits)
    err = scaled_rel_err(got, ref_f32)
    assert err <= FP16_TOL, f"{what}: scaled error {err:.3e} > {FP16_TOL}"
    d = ulp16_diff(got_bits, rne_bits)
    assert d.size == 0 or d.max() <= max_ulp, f"{what}: {d.max()} FP16 ulps from the oracle"
    frac = float((d != 0).mean()) if d.size else 0.0
    assert frac <= max_mismatch, f"{what}: {frac:.4%} of elements differ from the oracle's rounding"
    return err, frac


def assert_rope_close(got_bits, x_bits, ref_f32, what):
    """RoPE: the stated bar, plus an elementwise bound. The device's sin/cos and
    the C library's differ by a few FP32 ulps and the device fuses a*c - b*s
    into an FMA, so the FP32 result may move by ~1e-6 of the pair's magnitude
    before the one FP16 rounding (half an FP16 ulp of the result)."""
    got = oracle.widen(got_bits).astype(np.float64)
    ref = np.asarray(ref_f32, dtype=np.float64)
    err = scaled_rel_err(got, ref)
    assert err <= FP16_TOL, f"{what}: scaled error {err:.3e} > {FP16_TOL}"
    x = oracle.widen(x_bits).astype(np.float64)
    half = x.shape[-1] // 2
    mag = np.abs(x[..., :half]) + np.abs(x[..., half:])
    mag = np.concatenate([mag, mag], axis=-1)
    with np.errstate(over="ignore"):
        ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    bound = 0.5 * ulp + 1e-6 * mag + 2.0 ** -25
    worst = float(np.max(np.abs(got - ref) / bound))
    assert worst <= 1.0, f"{what}: {worst:.3f}x the elementwise bound"
    return err, worst
