"""Writes tests/golden/cpu_kernels_golden.npz from the COMPILED REFERENCE.

Run in the build container only (needs oracle/_ref/libvv_ref_cpu.so, which
oracle/Makefile compiles from the reference's src/cpu/cpu_kernels.c):

    python tests/golden/make_golden.py

The fixture holds inputs and the reference's outputs for its five layer
kernels (vv_rmsnorm_cpu, vv_rope_cpu, vv_swiglu_cpu, vv_residual_add_cpu,
vv_embedding_cpu) at small shapes. It also holds the int8 activation quantiser's outputs (vv_quant_act_q8_cpu)
in all four layouts. It is data only: no reference source text.
Inputs come from a local numpy generator and are stored in the file, so the
fixture does not depend on any generator staying stable.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402

f32p = C.POINTER(C.c_float)
i32p = C.POINTER(C.c_int32)


def p(a, ty):
    return a.ctypes.data_as(ty)


def main() -> None:
    ref = oracle.ref
    if ref is None:
        raise SystemExit("oracle/_ref/libvv_ref_cpu.so is missing: run `make -C oracle ref`")
    ref.vv_cpu_threads()
    rng = np.random.default_rng(20251125)
    out = {}

    # RMSNorm: Qwen2 width and a narrow row; weights ~N(1, 0.1) as FP16 bits.
    for tag, rows, n in (("rms_a", 3, 3584), ("rms_b", 5, 200)):
        x = rng.standard_normal((rows, n)).astype(np.float32)
        if tag == "rms_b":
            x[1] = 0.0                      # zero row
            x[2] *= 1e-3                    # eps-dominated row
            x[3] *= 300.0
        w = (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float16).view(np.uint16)
        y = np.empty_like(x)
        assert ref.vv_rmsnorm_cpu(p(x, f32p), w.ctypes.data, p(y, f32p), rows, n,
                                  C.c_float(1e-6)) == 0
        out[tag + "_x"], out[tag + "_w"], out[tag + "_y"] = x, w, y

    # RoPE: head_dim 128 / theta 1e6 at prefill and decode offsets; head_dim 64 / theta 1e4.
    for tag, rows, heads, hd, off, theta in (
            ("rope_a", 3, 4, 128, 0, 1e6), ("rope_b", 2, 2, 128, 8192, 1e6),
            ("rope_c", 2, 3, 128, 14447, 1e6), ("rope_d", 4, 2, 64, 913, 1e4)):
        x = rng.standard_normal((rows, heads, hd)).astype(np.float32)
        y = x.copy()
        assert ref.vv_rope_cpu(p(y, f32p), rows, heads, hd, off, C.c_float(theta)) == 0
        out[tag + "_x"], out[tag + "_y"] = x, y
        out[tag + "_meta"] = np.array([off, theta], dtype=np.float64)

    # SwiGLU: N(0, 2) plus the FP16 extremes and zeros.
    g = (2.0 * rng.standard_normal(4096)).astype(np.float32)
    u = (2.0 * rng.standard_normal(4096)).astype(np.float32)
    g[:8] = [0.0, -0.0, 65504.0, -65504.0, 88.0, -88.0, 1e-8, -104.0]
    u[8:12] = [0.0, -0.0, 65504.0, -65504.0]
    y = np.empty_like(g)
    assert ref.vv_swiglu_cpu(p(g, f32p), p(u, f32p), p(y, f32p), g.size) == 0
    out["swiglu_g"], out["swiglu_u"], out["swiglu_y"] = g, u, y

    # Residual add.
    a = rng.standard_normal(2048).astype(np.float32)
    b = rng.standard_normal(2048).astype(np.float32)
    s = a.copy()
    assert ref.vv_residual_add_cpu(p(s, f32p), p(b, f32p), s.size) == 0
    out["resid_a"], out["resid_b"], out["resid_y"] = a, b, s

    # Embedding: includes subnormal, inf and NaN bit patterns, first/last/duplicate ids.
    table = rng.integers(0, 65536, size=(37, 72), dtype=np.uint16)
    ids = np.array([0, 36, 5, 5, 17, 36, 0, 1], dtype=np.int32)
    e = np.empty((ids.size, 72), dtype=np.float32)
    assert ref.vv_embedding_cpu(table.ctypes.data, p(ids, i32p), p(e, f32p), ids.size, 72) == 0
    out["emb_table"], out["emb_ids"] = table, ids
    out["emb_y_bits"] = e.view(np.uint32)     # bits: NaN payloads survive the file

    # Int8 activation quantiser (src/cpu/cpu_int8.c), all four layouts.
    i8p = C.POINTER(C.c_int8)
    xq_in = (3.0 * rng.standard_normal((4, 256))).astype(np.float16).astype(np.float32)
    xq_in[1] = 0.0
    xq_in[2, :6] = [127.0, 0.5, 1.5, 2.5, -0.5, -126.5]
    xq_in[2, 6:] *= 0.01
    out["q8_x"] = xq_in
    for layout in range(4):
        q = np.empty((4, 256), np.int8)
        sx = np.empty(4, np.float32)
        xs = np.empty((4, 8), np.int32)
        assert ref.vv_quant_act_q8_cpu(p(xq_in, f32p), 4, 256, layout, q.ctypes.data_as(i8p),
                                       p(sx, f32p), p(xs, i32p)) == 0
        out[f"q8_q{layout}"], out[f"q8_sx{layout}"], out[f"q8_xs{layout}"] = q, sx, xs

    path = os.path.join(HERE, "cpu_kernels_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes; reference SIMD path:",
          ref.vv_cpu_simd_name().decode())


if __name__ == "__main__":
    main()
