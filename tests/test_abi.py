"""CPU checks of the drop-in boundary: the library loads, exports exactly the
symbols include/vibevoice_hip.h declares, and the argument checks that need no
GPU behave as the reference's do (NULL -> VV_ERR_NULL_PTR, empty -> VV_OK)."""
import os
import re
import subprocess

import pytest

from __graft_entry__ import ROOT, load_device

dev = load_device()
HEADER = os.path.join(ROOT, "include", "vibevoice_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vv_[a-z0-9_]+)\s*\(", text)))


def test_header_python_and_library_agree():
    declared = declared_symbols()
    assert len(declared) >= 51
    assert sorted(dev.SIGNATURES) == declared
    out = subprocess.check_output(["nm", "-D", "--defined-only", dev.LIB_PATH], text=True)
    exported = sorted(l.split()[-1] for l in out.splitlines() if " T " in l and " vv_" in l)
    assert exported == declared


def test_library_is_gfx950_only_and_does_not_link_the_oracle():
    out = subprocess.check_output(["ldd", dev.LIB_PATH], text=True)
    assert "libamdhip64" in out
    assert "oracle" not in out and "vv_ref" not in out and "gomp" not in out
    blob = open(dev.LIB_PATH, "rb").read()
    assert b"gfx950" in blob
    for other in (b"gfx942", b"gfx90a", b"sm_80"):
        assert other not in blob


def test_backend_name():
    assert dev.vv_dev_backend_name() == b"HIP"
    assert dev.vv_dev_host_shares_memory(0) is False


P = 0x1000   # a non-null, 16-byte aligned stand-in; never dereferenced by these calls


@pytest.mark.parametrize("call", [
    lambda: dev.vv_embedding_dev(None, P, P, 4, 3584, None),
    lambda: dev.vv_embedding_dev(P, None, P, 4, 3584, None),
    lambda: dev.vv_embedding_dev(P, P, None, 4, 3584, None),
    lambda: dev.vv_rmsnorm_dev(None, P, P, 4, 3584, 1e-6, None),
    lambda: dev.vv_rmsnorm_dev(P, None, P, 4, 3584, 1e-6, None),
    lambda: dev.vv_rmsnorm_dev(P, P, None, 4, 3584, 1e-6, None),
    lambda: dev.vv_rope_dev(None, 4, 28, 128, 0, None, 1e6, None),
    lambda: dev.vv_rope_qk_dev(None, None, 4, 28, 4, 128, 0, None, 1e6, None),
    lambda: dev.vv_swiglu_dev(None, P, P, 64, None),
    lambda: dev.vv_swiglu_dev(P, None, P, 64, None),
    lambda: dev.vv_swiglu_dev(P, P, None, 64, None),
    lambda: dev.vv_swiglu_fused_dev(None, P, 2, 64, None),
    lambda: dev.vv_residual_add_dev(None, P, 64, None),
    lambda: dev.vv_residual_add_dev(P, None, 64, None),
    lambda: dev.vv_bias_add_dev(None, P, 2, 64, None),
    lambda: dev.vv_add_rmsnorm_dev(None, P, P, P, 4, 3584, 1e-6, None),
    lambda: dev.vv_add_rmsnorm_dev(P, P, P, None, 4, 3584, 1e-6, None),
    lambda: dev.vv_embedding_rmsnorm_dev(P, None, P, P, P, 4, 3584, 1e-6, None),
    lambda: dev.vv_pos_add_dev(None, P, 1, None),
    lambda: dev.vv_dev_memcpy_d2d_at(P, P, 16, None, None),
    lambda: dev.vv_dev_alloc(None, 16),
    lambda: dev.vv_dev_memset_async(None, 0, 16, None),
    lambda: dev.vv_dev_event_record(None, None),
    lambda: dev.vv_dev_graph_launch(None, None),
])
def test_null_pointer_is_an_error_not_a_crash(call):
    assert call() == dev.VV_ERR_NULL_PTR


@pytest.mark.parametrize("call", [
    lambda: dev.vv_embedding_dev(P, P, P, 0, 3584, None),
    lambda: dev.vv_rmsnorm_dev(P, P, P, 0, 3584, 1e-6, None),
    lambda: dev.vv_rmsnorm_dev(P, P, P, -3, 3584, 1e-6, None),
    lambda: dev.vv_rope_dev(P, 0, 28, 128, 0, None, 1e6, None),
    lambda: dev.vv_rope_dev(P, 4, 0, 128, 0, None, 1e6, None),
    lambda: dev.vv_swiglu_dev(P, P, P, 0, None),
    lambda: dev.vv_swiglu_fused_dev(P, P, 0, 64, None),
    lambda: dev.vv_residual_add_dev(P, P, 0, None),
    lambda: dev.vv_bias_add_dev(P, P, 0, 64, None),
    lambda: dev.vv_add_rmsnorm_dev(P, P, P, P, 0, 3584, 1e-6, None),
    lambda: dev.vv_embedding_rmsnorm_dev(P, P, P, P, P, 0, 3584, 1e-6, None),
    lambda: dev.vv_dev_memcpy_d2d_at(P, P, 0, P, None),
    lambda: dev.vv_dev_free(None),
    lambda: dev.vv_dev_free_pinned(None),
    lambda: dev.vv_dev_stream_destroy(None),
    lambda: dev.vv_dev_event_destroy(None),
    lambda: dev.vv_dev_host_unregister(None),
])
def test_empty_work_is_ok_and_launches_nothing(call):
    assert call() == dev.VV_OK


def test_declined_arguments():
    assert dev.vv_rope_dev(P, 4, 2, 127, 0, None, 1e4, None) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_rope_dev(P, 4, 2, 1024, 0, None, 1e4, None) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_dev_graph_begin(None) == dev.VV_ERR_INVALID_ARG
    assert dev.vv_dev_host_register(P, 4096) == dev.VV_ERR_UNSUPPORTED
    assert dev.vv_dev_host_register(None, 4096) == dev.VV_ERR_NULL_PTR
    dev.vv_dev_graph_destroy(None)      # no-op, must not crash


def test_attention_host_queries():
    """The three attention queries run on the host and launch nothing."""
    AUTO, FA1, FA2, FI = 0, 1, 2, 3
    for requested in (AUTO, FA1, FA2, FI):
        for paged in (False, True):
            got = dev.vv_attn_resolve(requested, 0, paged, 28, 4, 128)
            assert got in (FA1, FA2, FI) and (requested in (AUTO, got) or paged)
            for fmt in (1, 3, 6):                                                  # FP8 and TurboQuant caches are served ...
                assert dev.vv_attn_resolve(requested, fmt, paged, 28, 4, 128) == got
                assert dev.vv_attn_resolve(requested, fmt, paged, 28, 4, 64) == FA1   # ... at head_dim 128 only
            assert dev.vv_attn_resolve(requested, 9, paged, 28, 4, 128) == FA1     # no such format
    assert dev.vv_attn_resolve(FA1, 0, True, 28, 4, 128) != FA1                    # fa1 never pages
    assert dev.vv_attn_scratch_bytes(28, 4, 128) == 28 * 2048 * 132 * 4      # decode slices / a split prefill's runs
    shapes = [dev.vv_attn_decode_shape(FA2, 28, 4, n) for n in range(1, 20000, 37)]
    assert shapes == sorted(shapes) and shapes[0] == 16 and shapes[-1] == 256
    assert set(shapes) <= {16, 32, 64, 128, 256}
    # still over the first 1024 positions, moving at 1025 (what the reference's own test asks of a backend)
    assert dev.vv_attn_decode_shape(FA2, 28, 4, 1) == dev.vv_attn_decode_shape(FA2, 28, 4, 1024) == 16
    assert dev.vv_attn_decode_shape(FA2, 28, 4, 1025) == dev.vv_attn_decode_shape(FA2, 28, 4, 2048) == 32
    assert dev.vv_gqa_decode_shape(1024) != dev.vv_gqa_decode_shape(1025)


# ── the whole seam ──────────────────────────────────────────────────────────

REF_HEADER = "/root/reference/include/vibevoice/device.h"


@pytest.mark.skipif(not os.path.exists(REF_HEADER), reason="reference tree not present")
def test_the_library_defines_every_symbol_of_the_reference_seam():
    text = re.sub(r"/\*.*?\*/", "", open(REF_HEADER).read(), flags=re.S)
    wanted = set(re.findall(r"^\s*(?:vv_status_t|int|size_t|void|bool|const char\*)\s+(vv_[a-z0-9_]+)\s*\(",
                            text, flags=re.M))
    out = subprocess.check_output(["nm", "-D", "--defined-only", dev.LIB_PATH], text=True)
    have = {l.split()[-1] for l in out.splitlines() if " T vv_" in l}
    assert not os.path.exists(os.path.join(os.path.dirname(dev.LIB_PATH), "libvibevoice_hip_unsupported.so"))
    assert len(wanted) >= 100 and not (wanted - have), sorted(wanted - have)
    # beyond device.h: the fused entry points, and the two kv_quant.h symbols
    # (kv_quant.h:96-101) the decoder links against
    assert have - wanted == {"vv_add_rmsnorm_dev", "vv_rope_qk_dev", "vv_bias_rope_qk_dev",
                             "vv_embedding_rmsnorm_dev", "vv_gemv_multi_dev", "vv_gemv_swiglu_dev",
                             "vv_kv_rotate_dev", "vv_kv_unrotate_dev", "vv_attn_decode_static",
                             "vv_rope_table_dev", "vv_gemm_bias_rope_dev", "vv_gemm_swiglu_dev",
                             "vv_gemm_qkv_rope_dev"}


HOST_ARCHIVE = os.path.join(ROOT, "oracle", "_ref", "host", "libvv_ref_host.a")


@pytest.mark.skipif(not os.path.exists(HOST_ARCHIVE), reason="oracle/_ref/host not built (needs the reference tree)")
def test_the_reference_host_code_links_against_this_library_alone():
    """The reference's host side (decoder, KV cache, pipeline, Conv-VAE front end, connectors, loaders ...), compiled
    where it lies into oracle/_ref/host/libvv_ref_host.a: every vv_ symbol it leaves undefined is one this library
    defines, so an engine links with -lvibevoice_hip and nothing else for the accelerator."""
    undefined = subprocess.run(["nm", "-u", HOST_ARCHIVE], capture_output=True, text=True).stdout
    defined = subprocess.run(["nm", "--defined-only", HOST_ARCHIVE], capture_output=True, text=True).stdout
    want = {l.split()[-1] for l in undefined.splitlines() if l.strip().startswith("U vv_")}
    have_host = {l.split()[-1] for l in defined.splitlines() if len(l.split()) == 3 and l.split()[-1].startswith("vv_")}
    need = want - have_host
    out = subprocess.check_output(["nm", "-D", "--defined-only", dev.LIB_PATH], text=True)
    ours = {l.split()[-1] for l in out.splitlines() if " T vv_" in l}
    assert len(need) >= 60 and not (need - ours), sorted(need - ours)
