"""ctypes view of libvibevoice_hip.so, one Python callable per C symbol.

Names, argument order and status codes are those of the C ABI
(include/vibevoice_hip.h, which mirrors the reference's
include/vibevoice/device.h): every function takes raw device addresses
(Python ints, e.g. ``tensor.data_ptr()``), a ``stream`` handle (0 = default
stream) and returns the ``vv_status_t`` integer. Nothing is converted, copied
or computed on the host.
"""
from __future__ import annotations

import ctypes as C
import os

VV_OK = 0
VV_ERR_INVALID_ARG = -1
VV_ERR_NULL_PTR = -2
VV_ERR_UNSUPPORTED = -7
VV_ERR_CUDA = -100
VV_ERR_CUDA_OOM = -101
VV_ERR_CUDA_LAUNCH = -102
VV_ATTN_DECODE_STATIC_MAX_Q_HEADS = 64    # include/vibevoice_hip.h

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib",
                        "libvibevoice_hip.so")

_vp, _i, _f, _sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t

class KvView(C.Structure):
    """vv_kv_view_t: one layer of a KV cache as the attention entry points see it."""
    _fields_ = [("k", C.c_void_p), ("v", C.c_void_p), ("k_meta", C.c_void_p),
                ("v_meta", C.c_void_p), ("page_table", C.c_void_p), ("format", C.c_int),
                ("n_kv_heads", C.c_int), ("head_dim", C.c_int)]


class SkinnyProj(C.Structure):
    """vv_skinny_proj_t: one projection of a small-M multi-projection launch."""
    _fields_ = [("w", C.c_void_p), ("scales", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p),
                ("N", C.c_int)]


class W4A16Proj(C.Structure):
    """vv_w4a16_proj_t: one projection of a fused W4A16 GEMV."""
    _fields_ = [("packed", C.c_void_p), ("sz", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p),
                ("N", C.c_int)]


class I8Proj(C.Structure):
    """vv_i8_proj_t: one projection of a shared-input int8 launch."""
    _fields_ = [("w", C.c_void_p), ("sw", C.c_void_p), ("sz", C.c_void_p), ("bias", C.c_void_p),
                ("y", C.c_void_p), ("N", C.c_int)]


VAE_MAX_ITEMS = 32


class VaeConvItem(C.Structure):
    """vv_vae_conv_item_t: one item's view of one convolution layer."""
    _fields_ = [("in_off", C.c_int64), ("out_off", C.c_int64), ("in_ptr", C.c_void_p), ("tail_in", C.c_void_p),
                ("tail_out", C.c_void_p), ("out_ptr", C.c_void_p), ("in_len", C.c_int), ("out_len", C.c_int),
                ("have", C.c_int), ("keep", C.c_int), ("out_ld", C.c_int), ("skip", C.c_int)]


class VaeConvDesc(C.Structure):
    """vv_vae_conv_desc_t: the items of a launch, passed by value to the kernels."""
    _fields_ = [("n", C.c_int), ("cap", C.c_int), ("it", VaeConvItem * VAE_MAX_ITEMS)]


class VaeRowSeg(C.Structure):
    _fields_ = [("row0", C.c_int), ("ld", C.c_int), ("dst", C.c_void_p)]


class VaeRows(C.Structure):
    """vv_vae_rows_t: where the rows of a connector GEMM go."""
    _fields_ = [("mode", C.c_int), ("n", C.c_int), ("seg", VaeRowSeg * VAE_MAX_ITEMS)]


# symbol -> (restype, argtypes); the complete export list of include/vibevoice_hip.h
SIGNATURES = {
    "vv_embedding_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "vv_rmsnorm_dev": (_i, [_vp, _vp, _vp, _i, _i, _f, _vp]),
    "vv_rope_dev": (_i, [_vp, _i, _i, _i, _i, _vp, _f, _vp]),
    "vv_swiglu_dev": (_i, [_vp, _vp, _vp, _i, _vp]),
    "vv_swiglu_fused_dev": (_i, [_vp, _vp, _i, _i, _vp]),
    "vv_residual_add_dev": (_i, [_vp, _vp, _i, _vp]),
    "vv_bias_add_dev": (_i, [_vp, _vp, _i, _i, _vp]),
    "vv_fp32_to_fp16_dev": (_i, [_vp, _vp, _i, _vp]),
    "vv_fp16_to_fp32_dev": (_i, [_vp, _vp, _i, _vp]),
    "vv_act_quant_dev": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "vv_rmsnorm_q8_dev": (_i, [_vp, _vp, _i, _i, _f, _i, _vp, _vp, _vp, _vp]),
    "vv_swiglu_q8_dev": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "vv_col_absmax_dev": (_i, [_vp, _i, _i, _vp, _vp]),
    "vv_gemm_fp16_dev": (_i, [_vp, _vp, _vp, _i, _i, _i, _f, _f, _vp]),
    "vv_gemm_fp16_tile_dev": (_i, [_vp, _vp, _vp, _i, _i, _i, _f, _f, _vp]),
    "vv_attn_resolve": (_i, [_i, _i, C.c_bool, _i, _i, _i]),
    "vv_attn_scratch_bytes": (C.c_size_t, [_i, _i, _i]),
    "vv_attn_decode_shape": (_i, [_i, _i, _i, _i]),
    "vv_attn_prefill": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, C.c_bool, _vp, _vp]),
    "vv_attn_decode": (_i, [_i, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp]),
    "vv_attn_decode_static": (_i, [_i, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "vv_kv_quant_store_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_bool, _i, _i, _i, _vp, _i, _i, _vp]),
    "vv_kv_dequant_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "vv_gqa_attention_decode_q_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp]),
    "vv_gqa_attention_prefill_q_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, C.c_bool, _i, _vp]),
    "vv_kv_rotate_dev": (_i, [_vp, _i, _i, _i, _vp]),
    "vv_kv_unrotate_dev": (_i, [_vp, _i, _i, _i, _vp]),
    "vv_kv_store_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_bool, _i, _i, _i, _vp, _i,
                            _i, _vp, _vp]),
    "vv_kv_page_map_dev": (_i, [_vp, _i, _i, _vp, _vp]),
    "vv_lm_head_gemv_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "vv_argmax_dev": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp]),
    "vv_skinny_linear_dev": (_i, [_vp, _i, _vp, _i, _i, _i, _f, _vp]),
    "vv_gemv_multi_dev": (_i, [_vp, _vp, _i, _i, _vp]),
    "vv_gemm_swiglu_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "vv_w4a16_gemv_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "vv_w4a16_gemv_multi_dev": (_i, [_vp, _vp, _i, _i, _i, _vp]),
    "vv_w4a16_gather_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "vv_w4a16_gemm_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, C.c_size_t, _i, _i, _i, _i, _vp]),
    "vv_w4a16_dequant_dev": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "vv_nf4_gemv_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    "vv_nf4_gemm_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "vv_dequant_nf4_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "vv_awq_gemv_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "vv_awq_gemm_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "vv_dequant_awq_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "vv_int8_gemv_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    "vv_int8_gemm_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "vv_dequant_int8_dev": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "vv_act_quant_i8_dev": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "vv_ternary_gemm_dev": (_i, [_vp, _vp, _vp, _vp, C.c_float, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "vv_i8_gemm_dev": (_i, [_vp, _vp, _vp, C.c_float, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "vv_i8s_requant_dev": (_i, [_vp, C.c_int64, _vp, _i, _vp, _vp, _vp]),
    "vv_i8_head_argmax_scratch_bytes": (C.c_size_t, [_i]),
    "vv_i8_head_argmax_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp]),
    "vv_vae_conv_dev": (_i, [_vp, _vp, C.c_int64, _vp, _vp, _vp, C.c_int64, _i, _i, _i, _i, C.c_bool, _vp]),
    "vv_vae_tail_dev": (_i, [_vp, _vp, C.c_int64, _i, _vp]),
    "vv_vae_rms_dev": (_i, [_vp, C.c_int64, C.c_int64, _i, C.c_float, _vp, _vp, _vp]),
    "vv_vae_mixer_dev": (_i, [_vp, _vp, _vp, C.c_int64, _vp, C.c_int64, _vp, _vp, _vp, _vp, _i, _i, _vp]),
    "vv_vae_im2col_dev": (_i, [_vp, _vp, C.c_int64, _i, _i, _i, C.c_int64, _i, _vp, C.c_int64, _vp]),
    "vv_vae_conv_gemm_dev": (_i, [_vp, _vp, _vp, C.c_int64, _vp, _vp, C.c_int64, _i, _i, C.c_int64, _i, _i, _vp]),
    "vv_vae_gemm_nn_dev": (_i, [_i, _vp, _vp, C.c_int64, _vp, C.c_int64, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "vv_vae_gemm_tn_dev": (_i, [_vp, C.c_int64, _vp, _vp, C.c_int64, _i, _i, _i, _vp, _vp, _vp]),
    "vv_vae_f32_to_f16_dev": (_i, [_vp, _vp, C.c_int64, _vp]),
    "vv_gemm_fp16_nn_dev": (_i, [_vp, _vp, _vp, _i, _i, _i, C.c_float, C.c_float, _vp]),
    "vv_gemm_cleanup": (None, []),
    "vv_w8a8_linear_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "vv_w4a8_linear_dev": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "vv_i8_linear_multi_dev": (_i, [_vp, _i, _vp, _vp, _i, _vp, _i, _i, _i, _i, _vp]),
    "vv_gemv_swiglu_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "vv_gqa_decode_scratch_bytes": (C.c_size_t, [_i, _i]),
    "vv_gqa_decode_shape": (_i, [_i]),
    "vv_gqa_attention_decode_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "vv_gqa_attention_prefill_cached_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, C.c_bool, _vp]),
    "vv_gqa_attention_prefill_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, C.c_bool, _vp]),
    "vv_add_rmsnorm_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _f, _vp]),
    "vv_rope_qk_dev": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp, _f, _vp]),
    "vv_bias_rope_qk_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _f, _vp]),
    "vv_rope_table_dev": (_i, [_vp, _i, _i, _i, _vp, _f, _vp]),
    "vv_gemm_bias_rope_dev": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "vv_gemm_qkv_rope_dev": (_i, [_vp] * 10 + [_i] * 5 + [_vp, _vp, _vp, _vp, _i, _vp, _vp]),
    "vv_embedding_rmsnorm_dev": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp]),
    "vv_dev_alloc": (_i, [C.POINTER(_vp), _sz]),
    "vv_dev_alloc_pinned": (_i, [C.POINTER(_vp), _sz]),
    "vv_dev_free": (_i, [_vp]),
    "vv_dev_free_pinned": (_i, [_vp]),
    "vv_dev_memcpy_h2d": (_i, [_vp, _vp, _sz, _vp]),
    "vv_dev_memcpy_d2h": (_i, [_vp, _vp, _sz, _vp]),
    "vv_dev_memcpy_d2d": (_i, [_vp, _vp, _sz, _vp]),
    "vv_dev_memcpy_d2d_at": (_i, [_vp, _vp, _sz, _vp, _vp]),
    "vv_dev_memset": (_i, [_vp, _i, _sz]),
    "vv_dev_memset_async": (_i, [_vp, _i, _sz, _vp]),
    "vv_dev_stream_create": (_i, [C.POINTER(_vp)]),
    "vv_dev_stream_create_background": (_i, [C.POINTER(_vp)]),
    "vv_dev_stream_destroy": (_i, [_vp]),
    "vv_dev_stream_sync": (_i, [_vp]),
    "vv_dev_set_device": (_i, [_i]),
    "vv_dev_get_device_info": (_i, [_i, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_i)]),
    "vv_dev_device_count": (_i, []),
    "vv_dev_get_device_name": (_i, [_i, C.c_char_p, _sz]),
    "vv_dev_host_shares_memory": (C.c_bool, [_i]),
    "vv_dev_memcpy_peer": (_i, [_vp, _i, _vp, _i, _sz, _vp]),
    "vv_dev_enable_peer": (_i, [_i, _i]),
    "vv_dev_event_create": (_i, [C.POINTER(_vp)]),
    "vv_dev_event_destroy": (_i, [_vp]),
    "vv_dev_event_record": (_i, [_vp, _vp]),
    "vv_dev_event_sync": (_i, [_vp]),
    "vv_dev_stream_wait_event": (_i, [_vp, _vp]),
    "vv_dev_host_register": (_i, [_vp, _sz]),
    "vv_dev_host_unregister": (_i, [_vp]),
    "vv_dev_backend_name": (C.c_char_p, []),
    "vv_dev_graph_begin": (_i, [_vp]),
    "vv_dev_graph_end": (_i, [_vp, C.POINTER(_vp)]),
    "vv_dev_graph_launch": (_i, [_vp, _vp]),
    "vv_dev_graph_destroy": (None, [_vp]),
    "vv_pos_add_dev": (_i, [_vp, _vp, _i, _vp]),
}


def _load() -> C.CDLL:
    # A process must hold ONE HIP runtime. PyTorch wheels bundle their own
    # libamdhip64.so.7; if this library were loaded first it would pull in the
    # system copy and a later `import torch` would bring a second one (observed:
    # a segmentation fault at torch's first device call). Importing torch first
    # makes the loader reuse torch's copy for this library (same SONAME). In a
    # process without torch the system runtime is used.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python vibevoice.c_amd/build.py` "
            "(there is no CPU fallback for the HIP backend)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the ABI lost a symbol
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()

# module-level callables with the C names
for _name in SIGNATURES:
    globals()[_name] = getattr(lib, _name)
del _name
