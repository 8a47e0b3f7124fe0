"""CPU checker for the HIP backend — TEST INFRASTRUCTURE ONLY.

``oracle.lib``   ctypes view of ``libvv_oracle.so`` (our restatement of the
                 reference's ``src/cpu`` layer kernels, ``vv_oracle.c``).
``oracle.ref``   ctypes view of ``_ref/libvv_ref_cpu.so`` — the reference's own
                 ``src/cpu/cpu_kernels.c`` compiled by ``oracle/Makefile`` — or
                 ``None`` when that file was not built.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` import this package. The shipped library never does.

All array arguments are C-contiguous numpy arrays; FP16 tensors travel as
``uint16`` bit patterns so that nothing is converted behind the caller's back.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvv_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libvv_ref_cpu.so")

_u16p = C.POINTER(C.c_uint16)
_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int32)


def build(force: bool = False) -> None:
    """Compile the checker (and ``_ref`` when the reference tree is present)."""
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "vv_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libvv_oracle.so"],
                              stdout=subprocess.DEVNULL)
    if force or not os.path.exists(_REF_PATH):
        subprocess.check_call(["make", "-C", _HERE, "ref"], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    lib.vvo_half_to_float.restype = C.c_float
    lib.vvo_half_to_float.argtypes = [C.c_uint16]
    lib.vvo_float_to_half_rne.restype = C.c_uint16
    lib.vvo_float_to_half_rne.argtypes = [C.c_float]
    lib.vvo_widen_f16.argtypes = [_u16p, _f32p, C.c_size_t]
    lib.vvo_narrow_f32_rne.argtypes = [_f32p, _u16p, C.c_size_t]
    lib.vvo_rmsnorm_f32.argtypes = [_f32p, _u16p, _f32p, C.c_int, C.c_int, C.c_float]
    lib.vvo_rope_f32.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]
    lib.vvo_swiglu_f32.argtypes = [_f32p, _f32p, _f32p, C.c_int]
    lib.vvo_residual_add_f32.argtypes = [_f32p, _f32p, C.c_int]
    lib.vvo_embedding_f32.argtypes = [_u16p, _i32p, _f32p, C.c_int, C.c_int]
    lib.vvo_rmsnorm_f16.argtypes = [_u16p, _u16p, _f32p, _u16p, C.c_int, C.c_int, C.c_float]
    lib.vvo_residual_add_f16.argtypes = [_u16p, _u16p, C.c_size_t]
    lib.vvo_add_rmsnorm_f16.argtypes = [_u16p, _u16p, _u16p, _f32p, _u16p,
                                        C.c_int, C.c_int, C.c_float]
    lib.vvo_rope_f16.argtypes = [_u16p, _f32p, _u16p, C.c_int, C.c_int, C.c_int,
                                 C.c_int, C.c_float]
    lib.vvo_swiglu_f16.argtypes = [_u16p, _u16p, _f32p, _u16p, C.c_size_t]
    lib.vvo_swiglu_fused_f16.argtypes = [_u16p, _f32p, _u16p, C.c_int, C.c_int]
    lib.vvo_embedding_f16.argtypes = [_u16p, _i32p, _u16p, C.c_int, C.c_int]
    lib.vvo_bias_add_f16.argtypes = [_u16p, _u16p, C.c_int, C.c_int]
    lib.vvo_fill_normal_f16.argtypes = [_u16p, C.c_size_t, C.c_uint64, C.c_double, C.c_double]
    lib.vvo_fill_normal_f32.argtypes = [_f32p, C.c_size_t, C.c_uint64, C.c_double, C.c_double]
    lib.vvo_fill_ids.argtypes = [_i32p, C.c_size_t, C.c_uint64, C.c_int32]
    lib.vvo_q8_pos.restype = C.c_int
    lib.vvo_q8_pos.argtypes = [C.c_int, C.c_int]
    lib.vvo_quant_act_q8.restype = C.c_int
    lib.vvo_quant_act_q8.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int8), _f32p, _i32p]
    lib.vvo_gemm_f16w.restype = C.c_int
    lib.vvo_gemm_f16w.argtypes = [_f32p, _u16p, _u16p, _f32p, C.c_int, C.c_int, C.c_int]
    lib.vvo_attention_prefill_f32.restype = C.c_int
    lib.vvo_attention_prefill_f32.argtypes = [_f32p, _f32p, _f32p, _f32p] + [C.c_int] * 7
    lib.vvo_w8a8_linear.restype = C.c_int
    lib.vvo_w8a8_linear.argtypes = [C.c_void_p, _f32p, C.c_void_p, _f32p, C.c_void_p, C.c_void_p, C.c_void_p,
                                    C.c_void_p, C.c_int, C.c_int, C.c_int]
    lib.vvo_w4a8_linear.restype = C.c_int
    lib.vvo_w4a8_linear.argtypes = [C.c_void_p, _f32p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p,
                                    C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int]
    lib.vvo_int4g_to_gpu_layout.restype = C.c_int
    lib.vvo_int4g_to_gpu_layout.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                            C.c_void_p]
    lib.vvo_int4g_dequant_f16.restype = C.c_int
    lib.vvo_int4g_dequant_f16.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]
    for name, args in (("vvo_fp8_encode", [_f32p, C.c_int, C.c_int, C.c_void_p]),
                       ("vvo_fp8_decode", [C.c_void_p, C.c_int, C.c_int, _f32p]),
                       ("vvo_kv_build_ref", [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
                       ("vvo_kv_store_fp8", [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p])):
        getattr(lib, name).restype = C.c_int
        getattr(lib, name).argtypes = args
    for name, args in (("vvo_nf4_dequant", [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]),
                       ("vvo_awq_dequant", [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                            C.c_void_p]),
                       ("vvo_int8_dequant", [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p])):
        getattr(lib, name).restype = C.c_int
        getattr(lib, name).argtypes = args
    for name, args in (("vvo_ternary_pack", [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]),
                       ("vvo_bn_act_quant", [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
                       ("vvo_ternary_linear", [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_int, C.c_int,
                                               C.c_int, C.c_void_p, C.c_void_p]),
                       ("vvo_i8_linear", [C.c_void_p, C.c_float, C.c_void_p, C.c_float, C.c_void_p, C.c_int, C.c_int,
                                          C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
                       ("vvo_i8s_requant", [C.c_void_p, C.c_int64, C.c_float, C.c_int, C.c_void_p, C.c_void_p]),
                       ("vvo_i8_head_argmax", [C.c_void_p, C.c_float, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                               C.c_void_p, C.c_void_p])):
        getattr(lib, name).restype = C.c_int
        getattr(lib, name).argtypes = args
    V, I64 = C.c_void_p, C.c_int64
    for name, args in (("vvo_vae_conv", [V, V, I64, V, V, V, I64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
                       ("vvo_vae_tail", [V, V, I64, C.c_int]),
                       ("vvo_vae_im2col", [V, V, I64, C.c_int, C.c_int, C.c_int, I64, C.c_int, V, I64]),
                       ("vvo_vae_conv_gemm", [V, V, I64, V, V, I64, C.c_int, C.c_int, C.c_int]),
                       ("vvo_vae_rms", [V, I64, I64, C.c_int, C.c_float, V, V]),
                       ("vvo_vae_mixer", [V, V, V, I64, V, I64, V, V, V, V, C.c_int, C.c_int]),
                       ("vvo_vae_gemm_nn", [C.c_int, V, V, I64, V, I64, C.c_int, C.c_int, C.c_int, V, V, V, V]),
                       ("vvo_vae_gemm_tn", [V, I64, V, V, I64, C.c_int, C.c_int, C.c_int, V, V])):
        getattr(lib, name).restype = C.c_int
        getattr(lib, name).argtypes = args
    lib.vvo_trunc_half.restype = C.c_uint16
    lib.vvo_trunc_half.argtypes = [C.c_float]
    for name, args in (("vvo_kv_bytes_per_vec", [C.c_int]),
                       ("vvo_kv_rotate", [C.c_void_p, C.c_int, C.c_int]),
                       ("vvo_kv_store_tq", [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
                       ("vvo_kv_unpack", [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
                       ("vvo_kv_dequant", [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p])):
        getattr(lib, name).restype = C.c_int
        getattr(lib, name).argtypes = args
    lib.vvo_argmax_first.restype = C.c_int
    lib.vvo_argmax_first.argtypes = [_f32p, C.c_int, C.POINTER(C.c_int32), _f32p]
    lib.vvo_threads.restype = C.c_int
    lib.vvo_set_threads.argtypes = [C.c_int]
    for name in ("vvo_rmsnorm_f32", "vvo_rope_f32", "vvo_swiglu_f32", "vvo_residual_add_f32",
                 "vvo_embedding_f32", "vvo_rmsnorm_f16", "vvo_residual_add_f16",
                 "vvo_add_rmsnorm_f16", "vvo_rope_f16", "vvo_swiglu_f16",
                 "vvo_swiglu_fused_f16", "vvo_embedding_f16", "vvo_bias_add_f16"):
        getattr(lib, name).restype = C.c_int
    return lib


def _load_ref():
    """The reference's compiled CPU kernels (include/vibevoice/cpu_kernels.h names)."""
    if not os.path.exists(_REF_PATH):
        return None
    ref = C.CDLL(_REF_PATH)
    vp = C.c_void_p
    ref.vv_rmsnorm_cpu.argtypes = [_f32p, vp, _f32p, C.c_int, C.c_int, C.c_float]
    ref.vv_rope_cpu.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]
    ref.vv_swiglu_cpu.argtypes = [_f32p, _f32p, _f32p, C.c_int]
    ref.vv_residual_add_cpu.argtypes = [_f32p, _f32p, C.c_int]
    ref.vv_embedding_cpu.argtypes = [vp, _i32p, _f32p, C.c_int, C.c_int]
    for name in ("vv_rmsnorm_cpu", "vv_rope_cpu", "vv_swiglu_cpu", "vv_residual_add_cpu",
                 "vv_embedding_cpu", "vv_cpu_threads", "vv_cpu_physical_cores"):
        getattr(ref, name).restype = C.c_int
    ref.vv_cpu_simd_name.restype = C.c_char_p
    ref.vv_gemm_f16w_cpu.restype = C.c_int
    ref.vv_gemm_f16w_cpu.argtypes = [_f32p, vp, vp, _f32p, C.c_int, C.c_int, C.c_int]
    ref.vv_attention_prefill_cpu.restype = C.c_int
    ref.vv_attention_prefill_cpu.argtypes = [_f32p, _f32p, _f32p, _f32p] + [C.c_int] * 6 + [C.c_bool]
    if hasattr(ref, "vv_w8a8_gemm_cpu"):
        ref.vv_w8a8_gemm_cpu.restype = C.c_int
        ref.vv_w8a8_gemm_cpu.argtypes = [C.c_void_p, _f32p, C.c_void_p, _f32p, C.c_void_p, _f32p,
                                         C.c_int, C.c_int, C.c_int]
    if hasattr(ref, "vv_w4a8_gemm_cpu"):
        ref.vv_w4a8_gemm_cpu.restype = C.c_int
        ref.vv_w4a8_gemm_cpu.argtypes = [C.c_void_p, _f32p, _i32p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                         C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int]
    if hasattr(ref, "vv_int4g_gemm_cpu"):
        ref.vv_int4g_gemm_cpu.restype = C.c_int
        ref.vv_int4g_gemm_cpu.argtypes = [_f32p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, _f32p,
                                          C.c_int, C.c_int, C.c_int, C.c_int]
    if hasattr(ref, "vv_nf4_gemm_cpu"):
        ref.vv_nf4_gemm_cpu.restype = C.c_int
        ref.vv_nf4_gemm_cpu.argtypes = [_f32p, C.c_void_p, C.c_void_p, C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int]
    if hasattr(ref, "vv_int8_gemm_cpu"):
        ref.vv_int8_gemm_cpu.restype = C.c_int
        ref.vv_int8_gemm_cpu.argtypes = [_f32p, C.c_void_p, C.c_void_p, C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int]
    for name, args in (("vv_ternary_pack", [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]),
                       ("vv_act_quant_i8_cpu", [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
                       ("vv_ternary_gemm_i32_cpu", [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int]),
                       ("vv_ternary_linear_cpu", [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_void_p,
                                                  C.c_int, C.c_int, C.c_int]),
                       ("vv_i8_gemm_i32_cpu", [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int]),
                       ("vv_i8_linear_cpu", [C.c_void_p, C.c_float, C.c_void_p, C.c_float, C.c_void_p, C.c_void_p,
                                             C.c_void_p, C.c_int, C.c_int, C.c_int]),
                       ("vv_i8s_requant_cpu", [C.c_void_p, C.c_int64, C.c_float, C.c_int, C.c_void_p, C.c_void_p]),
                       ("vv_i8_head_argmax_cpu", [C.c_void_p, C.c_float, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                                  C.c_void_p, C.c_void_p])):
        if hasattr(ref, name):
            getattr(ref, name).restype = C.c_int
            getattr(ref, name).argtypes = args
    if hasattr(ref, "vv_int4g_to_gpu_layout"):
        ref.vv_int4g_to_gpu_layout.restype = C.c_int
        ref.vv_int4g_to_gpu_layout.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                               C.c_void_p]
    if hasattr(ref, "vv_quant_act_q8_cpu"):
        ref.vv_quant_act_q8_cpu.restype = C.c_int
        ref.vv_quant_act_q8_cpu.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int8),
                                            _f32p, _i32p]
    return ref


lib = _load()
ref = _load_ref()


# ── small numpy conveniences ────────────────────────────────────────────────

def _p(a: np.ndarray, ty):
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    return a.ctypes.data_as(ty)


def _check(st: int, what: str) -> None:
    if st != 0:
        raise RuntimeError(f"oracle {what} returned status {st}")


def widen(h: np.ndarray) -> np.ndarray:
    """uint16 FP16 bits -> float32, exactly."""
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib.vvo_widen_f16(_p(h, _u16p), _p(out, _f32p), h.size)
    return out


def narrow(f: np.ndarray) -> np.ndarray:
    """float32 -> uint16 FP16 bits, round-to-nearest-even."""
    f = np.ascontiguousarray(f, dtype=np.float32)
    out = np.empty(f.shape, dtype=np.uint16)
    lib.vvo_narrow_f32_rne(_p(f, _f32p), _p(out, _u16p), f.size)
    return out


def normal_f16(shape, seed: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    out = np.empty(shape, dtype=np.uint16)
    lib.vvo_fill_normal_f16(_p(out, _u16p), out.size, seed, mean, std)
    return out


def normal_f32(shape, seed: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    out = np.empty(shape, dtype=np.float32)
    lib.vvo_fill_normal_f32(_p(out, _f32p), out.size, seed, mean, std)
    return out


def ids(n: int, seed: int, bound: int) -> np.ndarray:
    out = np.empty(n, dtype=np.int32)
    lib.vvo_fill_ids(_p(out, _i32p), n, seed, bound)
    return out


def rmsnorm_f32(x: np.ndarray, w16: np.ndarray, eps: float) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, n = x.shape
    out = np.empty_like(x)
    _check(lib.vvo_rmsnorm_f32(_p(x, _f32p), _p(w16, _u16p), _p(out, _f32p), rows, n, eps),
           "rmsnorm_f32")
    return out


def rope_f32(x: np.ndarray, position_offset: int, theta: float) -> np.ndarray:
    """x: [rows, n_heads, head_dim] float32; returns the rotated copy."""
    v = np.array(x, dtype=np.float32, order="C", copy=True)
    rows, n_heads, head_dim = v.shape
    _check(lib.vvo_rope_f32(_p(v, _f32p), rows, n_heads, head_dim, position_offset, theta),
           "rope_f32")
    return v


def swiglu_f32(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    gate = np.ascontiguousarray(gate, dtype=np.float32)
    up = np.ascontiguousarray(up, dtype=np.float32)
    out = np.empty_like(gate)
    _check(lib.vvo_swiglu_f32(_p(gate, _f32p), _p(up, _f32p), _p(out, _f32p), gate.size),
           "swiglu_f32")
    return out


def residual_add_f32(x: np.ndarray, y: np.ndarray) -> np.ndarray:
    v = np.array(x, dtype=np.float32, order="C", copy=True)
    y = np.ascontiguousarray(y, dtype=np.float32)
    _check(lib.vvo_residual_add_f32(_p(v, _f32p), _p(y, _f32p), v.size), "residual_add_f32")
    return v


def embedding_f32(table16: np.ndarray, tok: np.ndarray) -> np.ndarray:
    hidden = table16.shape[1]
    tok = np.ascontiguousarray(tok, dtype=np.int32)
    out = np.empty((tok.size, hidden), dtype=np.float32)
    _check(lib.vvo_embedding_f32(_p(table16, _u16p), _p(tok, _i32p), _p(out, _f32p),
                                 tok.size, hidden), "embedding_f32")
    return out


def rmsnorm_f16(x16: np.ndarray, w16: np.ndarray, eps: float):
    """-> (ref float32, rne uint16) for the vv_rmsnorm_dev contract."""
    rows, n = x16.shape
    ref_ = np.empty((rows, n), dtype=np.float32)
    rne = np.empty((rows, n), dtype=np.uint16)
    _check(lib.vvo_rmsnorm_f16(_p(x16, _u16p), _p(w16, _u16p), _p(ref_, _f32p), _p(rne, _u16p),
                               rows, n, eps), "rmsnorm_f16")
    return ref_, rne


def residual_add_f16(x16: np.ndarray, y16: np.ndarray) -> np.ndarray:
    v = np.array(x16, dtype=np.uint16, order="C", copy=True)
    _check(lib.vvo_residual_add_f16(_p(v, _u16p), _p(y16, _u16p), v.size), "residual_add_f16")
    return v


def add_rmsnorm_f16(res16: np.ndarray, x16: np.ndarray, w16: np.ndarray, eps: float):
    """-> (updated residual uint16, normed ref float32, normed rne uint16)."""
    rows, n = res16.shape
    r = np.array(res16, dtype=np.uint16, order="C", copy=True)
    ref_ = np.empty((rows, n), dtype=np.float32)
    rne = np.empty((rows, n), dtype=np.uint16)
    _check(lib.vvo_add_rmsnorm_f16(_p(r, _u16p), _p(x16, _u16p), _p(w16, _u16p), _p(ref_, _f32p),
                                   _p(rne, _u16p), rows, n, eps), "add_rmsnorm_f16")
    return r, ref_, rne


def rope_f16(x16: np.ndarray, position_offset: int, theta: float):
    rows, n_heads, head_dim = x16.shape
    ref_ = np.empty(x16.shape, dtype=np.float32)
    rne = np.empty(x16.shape, dtype=np.uint16)
    _check(lib.vvo_rope_f16(_p(x16, _u16p), _p(ref_, _f32p), _p(rne, _u16p), rows, n_heads,
                            head_dim, position_offset, theta), "rope_f16")
    return ref_, rne


def swiglu_f16(g16: np.ndarray, u16: np.ndarray):
    ref_ = np.empty(g16.shape, dtype=np.float32)
    rne = np.empty(g16.shape, dtype=np.uint16)
    _check(lib.vvo_swiglu_f16(_p(g16, _u16p), _p(u16, _u16p), _p(ref_, _f32p), _p(rne, _u16p),
                              g16.size), "swiglu_f16")
    return ref_, rne


def swiglu_fused_f16(gu16: np.ndarray):
    rows, two_inter = gu16.shape
    inter = two_inter // 2
    ref_ = np.empty((rows, inter), dtype=np.float32)
    rne = np.empty((rows, inter), dtype=np.uint16)
    _check(lib.vvo_swiglu_fused_f16(_p(gu16, _u16p), _p(ref_, _f32p), _p(rne, _u16p),
                                    rows, inter), "swiglu_fused_f16")
    return ref_, rne


def embedding_f16(table16: np.ndarray, tok: np.ndarray) -> np.ndarray:
    hidden = table16.shape[1]
    tok = np.ascontiguousarray(tok, dtype=np.int32)
    out = np.empty((tok.size, hidden), dtype=np.uint16)
    _check(lib.vvo_embedding_f16(_p(table16, _u16p), _p(tok, _i32p), _p(out, _u16p),
                                 tok.size, hidden), "embedding_f16")
    return out


def bias_add_f16(out16: np.ndarray, bias16: np.ndarray) -> np.ndarray:
    v = np.array(out16, dtype=np.uint16, order="C", copy=True)
    M, N = v.shape
    _check(lib.vvo_bias_add_f16(_p(v, _u16p), _p(bias16, _u16p), M, N), "bias_add_f16")
    return v


def quant_act_q8(x: np.ndarray, layout: int, want_xsum: bool = True):
    """float32 [M,K] -> (int8 [M,K] in `layout`, float32 scale [M], int32 xsum [M,K/32] or None)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    xq = np.empty((M, K), dtype=np.int8)
    sx = np.empty(M, dtype=np.float32)
    xs = np.empty((M, K // 32), dtype=np.int32) if want_xsum else None
    _check(lib.vvo_quant_act_q8(_p(x, _f32p), M, K, layout, xq.ctypes.data_as(C.POINTER(C.c_int8)),
                                _p(sx, _f32p), _p(xs, _i32p) if want_xsum else None),
           "quant_act_q8")
    return xq, sx, xs


def gemm_f16w(x: np.ndarray, w16: np.ndarray, bias16=None) -> np.ndarray:
    """float32 x [M,K] times FP16 weight bits [N,K] (transposed) + FP16 bias bits [N]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    N = w16.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    _check(lib.vvo_gemm_f16w(_p(x, _f32p), _p(w16, _u16p),
                             _p(bias16, _u16p) if bias16 is not None else None,
                             _p(out, _f32p), M, N, K), "gemm_f16w")
    return out


def attention_prefill_f32(q, k, v, q_offset: int, kv_len: int, causal: bool = True) -> np.ndarray:
    """q [rows, n_q, hd], k/v [kv_len, n_kv, hd] float32 -> out like q."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    rows, n_q, hd = q.shape
    out = np.empty_like(q)
    _check(lib.vvo_attention_prefill_f32(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(out, _f32p),
                                         n_q, k.shape[1], hd, rows, q_offset, kv_len, int(causal)),
           "attention_prefill_f32")
    return out


def argmax_first(logits: np.ndarray):
    """(token, value): the first maximum of an in-order scan over float32 logits."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    tok, val = C.c_int32(), C.c_float()
    _check(lib.vvo_argmax_first(_p(logits, _f32p), logits.size, C.byref(tok), C.byref(val)), "argmax_first")
    return int(tok.value), float(val.value)


def w8a8_linear(xq, sx, w, sw, bias16=None, res16=None):
    """int8 [M,K] x int8 [N,K]^T with per-row scales -> (float32 [M,N], FP16 bits [M,N])."""
    xq, w = np.ascontiguousarray(xq, np.int8), np.ascontiguousarray(w, np.int8)
    sx, sw = np.ascontiguousarray(sx, np.float32), np.ascontiguousarray(sw, np.float32)
    M, K = xq.shape
    N = w.shape[0]
    f32, f16 = np.empty((M, N), np.float32), np.empty((M, N), np.uint16)
    ptr = lambda a: a.ctypes.data if a is not None else None
    if bias16 is not None:
        bias16 = np.ascontiguousarray(bias16, np.uint16)
    if res16 is not None:
        res16 = np.ascontiguousarray(res16, np.uint16)
    _check(lib.vvo_w8a8_linear(xq.ctypes.data, _p(sx, _f32p), w.ctypes.data, _p(sw, _f32p), ptr(bias16),
                               ptr(res16), f32.ctypes.data, f16.ctypes.data, M, N, K), "w8a8_linear")
    return f32, f16


def w4a8_linear(xq, sx, packed, scales16, zeros, G, bias16=None, res16=None):
    """int8 [M,K] (column order) x INT4G codes [N,K/2] (row-major, high nibble = even column) with FP16
    group scales [N,K/G] and integer zero points -> (float32 [M,N], FP16 bits [M,N])."""
    xq = np.ascontiguousarray(xq, np.int8)
    packed = np.ascontiguousarray(packed, np.uint8)
    scales16, zeros = np.ascontiguousarray(scales16, np.uint16), np.ascontiguousarray(zeros, np.uint8)
    sx = np.ascontiguousarray(sx, np.float32)
    M, K = xq.shape
    N = packed.shape[0]
    f32, f16 = np.empty((M, N), np.float32), np.empty((M, N), np.uint16)
    ptr = lambda a: a.ctypes.data if a is not None else None
    if bias16 is not None:
        bias16 = np.ascontiguousarray(bias16, np.uint16)
    if res16 is not None:
        res16 = np.ascontiguousarray(res16, np.uint16)
    _check(lib.vvo_w4a8_linear(xq.ctypes.data, _p(sx, _f32p), packed.ctypes.data, scales16.ctypes.data,
                               zeros.ctypes.data, G, ptr(bias16), ptr(res16), f32.ctypes.data, f16.ctypes.data,
                               M, N, K), "w4a8_linear")
    return f32, f16


def int4g_to_gpu_layout(packed, scales16, zeros, G):
    """Row-major INT4G codes -> (codes in the accelerator layout, half2 {scale, zero} bits [N,K/G,2])."""
    out = np.array(packed, dtype=np.uint8, order="C", copy=True)
    scales16, zeros = np.ascontiguousarray(scales16, np.uint16), np.ascontiguousarray(zeros, np.uint8)
    N, K = out.shape[0], out.shape[1] * 2
    sz = np.empty((N, K // G, 2), np.uint16)
    _check(lib.vvo_int4g_to_gpu_layout(out.ctypes.data, scales16.ctypes.data, zeros.ctypes.data, N, K, G,
                                       sz.ctypes.data), "int4g_to_gpu_layout")
    return out, sz


def int4g_dequant_f16(packed, scales16, zeros, G):
    """Row-major INT4G codes [N,K/2] -> FP16 bits [N,K] of (q - z) * s, rounded once."""
    packed = np.ascontiguousarray(packed, np.uint8)
    scales16, zeros = np.ascontiguousarray(scales16, np.uint16), np.ascontiguousarray(zeros, np.uint8)
    N, K = packed.shape[0], packed.shape[1] * 2
    out = np.empty((N, K), np.uint16)
    _check(lib.vvo_int4g_dequant_f16(packed.ctypes.data, scales16.ctypes.data, zeros.ctypes.data, N, K, G,
                                     out.ctypes.data), "int4g_dequant_f16")
    return out


def nf4_dequant(packed, scales16):
    """NF4 codes [N, K/2] and FP16 absmax bits per 64 flat elements -> (FP16 bits, FP32 values), both [N, K]."""
    packed = np.ascontiguousarray(packed, np.uint8)
    scales16 = np.ascontiguousarray(scales16, np.uint16)
    N, K = packed.shape[0], packed.shape[1] * 2
    assert scales16.size * 64 == N * K
    o16, o32 = np.empty((N, K), np.uint16), np.empty((N, K), np.float32)
    _check(lib.vvo_nf4_dequant(packed.ctypes.data, scales16.ctypes.data, N * K, o16.ctypes.data, o32.ctypes.data),
           "nf4_dequant")
    return o16, o32


def awq_dequant(packed, scales16, mins16, G: int):
    """INT4 codes [N, K/2] with FP16 scale and min bits [N, K/G] -> (FP16 bits, FP32 values) of q * scale + min."""
    packed = np.ascontiguousarray(packed, np.uint8)
    scales16, mins16 = np.ascontiguousarray(scales16, np.uint16), np.ascontiguousarray(mins16, np.uint16)
    N, K = packed.shape[0], packed.shape[1] * 2
    o16, o32 = np.empty((N, K), np.uint16), np.empty((N, K), np.float32)
    _check(lib.vvo_awq_dequant(packed.ctypes.data, scales16.ctypes.data, mins16.ctypes.data, N, K, G, o16.ctypes.data,
                               o32.ctypes.data), "awq_dequant")
    return o16, o32


def int8_dequant(q, scales):
    """int8 codes [N, K] with an FP32 scale per row -> (FP16 bits, FP32 values) of q * scale."""
    q = np.ascontiguousarray(q, np.int8)
    scales = np.ascontiguousarray(scales, np.float32)
    N, K = q.shape
    o16, o32 = np.empty((N, K), np.uint16), np.empty((N, K), np.float32)
    _check(lib.vvo_int8_dequant(q.ctypes.data, scales.ctypes.data, N, K, o16.ctypes.data, o32.ctypes.data),
           "int8_dequant")
    return o16, o32


# ── Conv-VAE encoder ops: thin views of the C functions ─────────────────────
# The descriptor mirrors include/vibevoice/device.h:733-755 field for field, so
# one ctypes layout serves the oracle (host pointers) and the device library.

VAE_MAX_ITEMS = 32


class VaeConvItem(C.Structure):
    _fields_ = [("in_off", C.c_int64), ("out_off", C.c_int64), ("in_ptr", C.c_void_p), ("tail_in", C.c_void_p),
                ("tail_out", C.c_void_p), ("out_ptr", C.c_void_p), ("in_len", C.c_int), ("out_len", C.c_int),
                ("have", C.c_int), ("keep", C.c_int), ("out_ld", C.c_int), ("skip", C.c_int)]


class VaeConvDesc(C.Structure):
    _fields_ = [("n", C.c_int), ("cap", C.c_int), ("it", VaeConvItem * VAE_MAX_ITEMS)]


class VaeRowSeg(C.Structure):
    _fields_ = [("row0", C.c_int), ("ld", C.c_int), ("dst", C.c_void_p)]


class VaeRows(C.Structure):
    _fields_ = [("mode", C.c_int), ("n", C.c_int), ("seg", VaeRowSeg * VAE_MAX_ITEMS)]


def _hp(a):
    """Host address of a numpy array (or None)."""
    return a.ctypes.data if a is not None else None


def vae_conv(desc, x, ld_in, w, b, y, ld_out, in_ch, out_ch, k, stride, transposed=False):
    _check(lib.vvo_vae_conv(C.addressof(desc), _hp(x), ld_in, _hp(w), _hp(b), _hp(y), ld_out, in_ch, out_ch, k, stride,
                            int(transposed)), "vae_conv")


def vae_tail(desc, x, ld_in, in_ch):
    _check(lib.vvo_vae_tail(C.addressof(desc), _hp(x), ld_in, in_ch), "vae_tail")


def vae_im2col(desc, x, ld_in, in_ch, k, stride, p0, pc, col, ldcol):
    _check(lib.vvo_vae_im2col(C.addressof(desc), _hp(x), ld_in, in_ch, k, stride, p0, pc, _hp(col), ldcol), "vae_im2col")


def vae_conv_gemm(w, col, ldcol, b, y, ld_out, out_ch, K, pc):
    _check(lib.vvo_vae_conv_gemm(_hp(w), _hp(col), ldcol, _hp(b), _hp(y), ld_out, out_ch, K, pc), "vae_conv_gemm")


def vae_rms(x, ld, T, Cn, eps, rinv, desc=None):
    _check(lib.vvo_vae_rms(_hp(x), ld, T, Cn, eps, _hp(rinv), C.addressof(desc) if desc is not None else None), "vae_rms")


def vae_mixer(desc, xin, xout, ld, rinv, T_total, nw, cw, cb, gamma, Cn, k):
    _check(lib.vvo_vae_mixer(C.addressof(desc), _hp(xin), _hp(xout), ld, _hp(rinv), T_total, _hp(nw), _hp(cw), _hp(cb),
                             _hp(gamma), Cn, k), "vae_mixer")


def vae_gemm_nn(epilogue, A, B, ldb, Cm, ldc, M, K, P, bias=None, gamma=None, rinv=None, nw=None):
    _check(lib.vvo_vae_gemm_nn(epilogue, _hp(A), _hp(B), ldb, _hp(Cm), ldc, M, K, P, _hp(bias), _hp(gamma), _hp(rinv),
                               _hp(nw)), "vae_gemm_nn")


def vae_gemm_tn(A, lda, B, Cm, ldc, M, N, K, bias=None, rows=None):
    _check(lib.vvo_vae_gemm_tn(_hp(A), lda, _hp(B), _hp(Cm), ldc, M, N, K, _hp(bias),
                               C.addressof(rows) if rows is not None else None), "vae_gemm_tn")


def trunc_half(f: float) -> int:
    return int(lib.vvo_trunc_half(float(f)))


def ternary_pack(t) -> np.ndarray:
    """Ternary values {-1, 0, 1} [N, K] (K % 128 == 0) -> the I2_S bytes [N, K/4]."""
    t = np.ascontiguousarray(t, np.int8)
    N, K = t.shape
    codes = np.empty((N, K // 4), np.uint8)
    _check(lib.vvo_ternary_pack(t.ctypes.data, N, K, codes.ctypes.data), "ternary_pack")
    return codes


def bn_act_quant(x):
    """FP32 rows [M, K] -> (int8 codes [M, K], multiplier [M], row sums of the codes [M])."""
    x = np.ascontiguousarray(x, np.float32)
    M, K = x.shape
    q, s, sm = np.empty((M, K), np.int8), np.empty(M, np.float32), np.empty(M, np.int32)
    _check(lib.vvo_bn_act_quant(x.ctypes.data, M, K, q.ctypes.data, s.ctypes.data, sm.ctypes.data), "bn_act_quant")
    return q, s, sm


def ternary_linear(q, x_scale, codes, w_scale: float, bias=None):
    """int8 rows [M, K] against I2_S codes [N, K/4] -> (int32 sums [M, N], FP32 y [M, N])."""
    q, codes = np.ascontiguousarray(q, np.int8), np.ascontiguousarray(codes, np.uint8)
    x_scale = np.ascontiguousarray(x_scale, np.float32)
    M, K = q.shape
    N = codes.shape[0]
    if bias is not None:
        bias = np.ascontiguousarray(bias, np.float32)
    acc, y = np.empty((M, N), np.int32), np.empty((M, N), np.float32)
    _check(lib.vvo_ternary_linear(q.ctypes.data, x_scale.ctypes.data, codes.ctypes.data, w_scale,
                                  bias.ctypes.data if bias is not None else None, M, N, K, acc.ctypes.data,
                                  y.ctypes.data), "ternary_linear")
    return acc, y


def i8_linear(a, a_scale: float, w, w_scale: float, bias=None):
    """int8 rows [M, K] against int8 weights [N, K] -> (int32 sums, FP32 y, max |y|)."""
    a, w = np.ascontiguousarray(a, np.int8), np.ascontiguousarray(w, np.int8)
    M, K = a.shape
    N = w.shape[0]
    if bias is not None:
        bias = np.ascontiguousarray(bias, np.float32)
    acc, y, am = np.empty((M, N), np.int32), np.empty((M, N), np.float32), np.zeros(1, np.float32)
    _check(lib.vvo_i8_linear(a.ctypes.data, a_scale, w.ctypes.data, w_scale, bias.ctypes.data if bias is not None else None,
                             M, N, K, acc.ctypes.data, y.ctypes.data, am.ctypes.data), "i8_linear")
    return acc, y, float(am[0])


def i8s_requant(y, absmax: float, relu: bool):
    """FP32 values -> (int8 codes of the same shape, the multiplier 127 / absmax)."""
    y = np.ascontiguousarray(y, np.float32)
    q, inv = np.empty(y.shape, np.int8), np.zeros(1, np.float32)
    _check(lib.vvo_i8s_requant(y.ctypes.data, y.size, absmax, int(relu), q.ctypes.data, inv.ctypes.data), "i8s_requant")
    return q, float(inv[0])


def i8_head_argmax(q, scale: float, w, w_scale):
    """int8 activation [K] against int8 rows [V, K] with a scale per row -> (token, its logit)."""
    q, w = np.ascontiguousarray(q, np.int8), np.ascontiguousarray(w, np.int8)
    w_scale = np.ascontiguousarray(w_scale, np.float32)
    V, K = w.shape
    tok, val = np.zeros(1, np.int32), np.zeros(1, np.float32)
    _check(lib.vvo_i8_head_argmax(q.ctypes.data, scale, w.ctypes.data, w_scale.ctypes.data, V, K, tok.ctypes.data,
                                  val.ctypes.data), "i8_head_argmax")
    return int(tok[0]), float(val[0])


def fp8_encode(x, e5m2: bool) -> np.ndarray:
    """float32 values -> FP8 codes (uint8, same shape)."""
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    _check(lib.vvo_fp8_encode(_p(x, _f32p), x.size, int(e5m2), out.ctypes.data), "fp8_encode")
    return out


def fp8_decode(codes, e5m2: bool) -> np.ndarray:
    """FP8 codes -> float32 values (same shape)."""
    codes = np.ascontiguousarray(codes, np.uint8)
    out = np.empty(codes.shape, np.float32)
    _check(lib.vvo_fp8_decode(codes.ctypes.data, codes.size, int(e5m2), _p(out, _f32p)), "fp8_decode")
    return out


def kv_build_ref(k16) -> np.ndarray:
    """FP16 keys [n_pos, n_kv_heads, head_dim] -> their per-head mean, FP16 bits [n_kv_heads, head_dim]."""
    k16 = np.ascontiguousarray(k16, np.uint16)
    n_pos, nkv, hd = k16.shape
    ref = np.empty((nkv, hd), np.uint16)
    _check(lib.vvo_kv_build_ref(k16.ctypes.data, n_pos, nkv, hd, ref.ctypes.data), "kv_build_ref")
    return ref


def kv_store_fp8(src16, ref16, e5m2: bool) -> np.ndarray:
    """FP16 vectors [n_pos, n_kv_heads, head_dim] (minus ref16 [n_kv_heads, head_dim] when given) -> FP8 codes."""
    src16 = np.ascontiguousarray(src16, np.uint16)
    n_pos, nkv, hd = src16.shape
    if ref16 is not None:
        ref16 = np.ascontiguousarray(ref16, np.uint16)
    out = np.empty((n_pos, nkv, hd), np.uint8)
    _check(lib.vvo_kv_store_fp8(src16.ctypes.data, ref16.ctypes.data if ref16 is not None else None, n_pos, nkv, hd,
                                int(e5m2), out.ctypes.data), "kv_store_fp8")
    return out


def kv_bytes_per_vec(fmt: int) -> int:
    return lib.vvo_kv_bytes_per_vec(fmt)


def kv_rotate(x16, inverse: bool = False) -> np.ndarray:
    """FP16 bits [..., 128] -> the randomised Hadamard transform (or its inverse) of every vector."""
    out = np.array(x16, dtype=np.uint16, order="C", copy=True)
    _check(lib.vvo_kv_rotate(out.ctypes.data, out.size // 128, int(inverse)), "kv_rotate")
    return out


def kv_store_tq(src16, ref16, fmt: int):
    """FP16 vectors [n_pos, n_kv_heads, 128] -> (codes uint8 [n_pos, n_kv_heads, bytes], RMS FP16 bits [n_pos, n_kv_heads])."""
    src16 = np.ascontiguousarray(src16, np.uint16)
    n_pos, nkv, hd = src16.shape
    assert hd == 128
    if ref16 is not None:
        ref16 = np.ascontiguousarray(ref16, np.uint16)
    store = np.empty((n_pos, nkv, kv_bytes_per_vec(fmt)), np.uint8)
    meta = np.empty((n_pos, nkv), np.uint16)
    _check(lib.vvo_kv_store_tq(src16.ctypes.data, ref16.ctypes.data if ref16 is not None else None, n_pos, nkv, fmt,
                               store.ctypes.data, meta.ctypes.data), "kv_store_tq")
    return store, meta


def kv_unpack(store, meta16, fmt: int) -> np.ndarray:
    """Codes [n_pos, n_kv_heads, bytes] (+ RMS for TurboQuant) -> FP16 bits [n_pos, n_kv_heads, 128] in the space
    they were stored in (TurboQuant: rotated): the values attention over the cache multiplies with."""
    store = np.ascontiguousarray(store, np.uint8)
    n_pos, nkv = store.shape[:2]
    if meta16 is not None:
        meta16 = np.ascontiguousarray(meta16, np.uint16)
    out = np.empty((n_pos, nkv, 128), np.uint16)
    _check(lib.vvo_kv_unpack(store.ctypes.data, meta16.ctypes.data if meta16 is not None else None, n_pos * nkv, fmt,
                             out.ctypes.data), "kv_unpack")
    return out


def kv_dequant(store, meta16, ref16, fmt: int) -> np.ndarray:
    """Codes [n_pos, n_kv_heads, bytes] (+ RMS for TurboQuant) -> FP16 bits [n_pos, n_kv_heads, 128] in the original
    space (TurboQuant: un-rotated), plus the reference key when given."""
    store = np.ascontiguousarray(store, np.uint8)
    n_pos, nkv = store.shape[:2]
    if meta16 is not None:
        meta16 = np.ascontiguousarray(meta16, np.uint16)
    if ref16 is not None:
        ref16 = np.ascontiguousarray(ref16, np.uint16)
    out = np.empty((n_pos, nkv, 128), np.uint16)
    _check(lib.vvo_kv_dequant(store.ctypes.data, meta16.ctypes.data if meta16 is not None else None,
                              ref16.ctypes.data if ref16 is not None else None, n_pos, nkv, fmt, out.ctypes.data),
           "kv_dequant")
    return out
