"""Runs the plain-C ABI program (tests/c/abi_layer_ops.c) on the GPU: the
library linked and called from C, with the system HIP runtime and no Python or
torch in the process, the way the reference's C engine would use it."""
import os
import subprocess

import pytest

import functools

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "c", "abi_layer_ops")
# Written by __graft_entry__.build() when it compiled the reference's test programs (oracle/Makefile,
# which needs the reference tree). It travels with the built programs, so where it is present a missing
# program is a broken build or a lost file and fails loudly; a checkout built without the reference
# tree has neither and skips.
REF_MARKER = os.path.join(os.path.dirname(HERE), "oracle", "ref_built.marker")


def needs_ref_program(path):
    def wrap(fn):
        @functools.wraps(fn)
        def run(*a, **kw):
            if not os.path.exists(path):
                rel = os.path.relpath(path, os.path.dirname(HERE))
                if os.path.exists(REF_MARKER):
                    pytest.fail(f"{rel} is missing although the reference's test programs were built "
                                f"({os.path.relpath(REF_MARKER, os.path.dirname(HERE))} is present)")
                pytest.skip(f"{rel} not built (needs the reference tree)")
            return fn(*a, **kw)
        return run
    return wrap


@pytest.mark.gpu
def test_c_program_links_and_passes():
    assert os.path.exists(EXE), "tests/c/abi_layer_ops is not built: run __graft_entry__.build()"
    res = subprocess.run([EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-4000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-2000:]
    assert "all C ABI checks passed" in res.stdout and "FAIL" not in res.stdout


def test_c_program_is_built_against_the_public_header():
    src = open(os.path.join(HERE, "c", "abi_layer_ops.c")).read()
    assert '#include "vibevoice_hip.h"' in src and "hip_runtime" not in src


REF_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_device_memory_hip")


@pytest.mark.gpu
@needs_ref_program(REF_EXE)
def test_reference_own_device_memory_test_passes_on_this_backend():
    """The reference's tests/test_device_memory.c, compiled unmodified by
    oracle/Makefile and linked against libvibevoice_hip.so: copies, fills,
    device-side index, events, pinned memory, graph capture/replay/break."""
    res = subprocess.run([REF_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-1000:])
    assert res.returncode == 0, res.stdout[-2000:]
    assert "all device memory checks passed" in res.stdout and "FAIL" not in res.stdout


LAYER_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_prefill_append_hip")


@pytest.mark.gpu
@needs_ref_program(LAYER_EXE)
def test_reference_layer_runner_passes_on_this_backend():
    """The reference's tests/test_prefill_append.c with the reference's own
    decoder and KV cache (compiled unmodified by oracle/Makefile) driving this
    backend: a 2-layer dense model, one-shot prefill vs prefill + decode step +
    prefill on top of the cache, and accelerator vs CPU hidden states. Every op
    of a dense layer goes through libvibevoice_hip.so: RMSNorm, the GEMMs and
    bias adds, RoPE, the FP16 KV append, prefill and decode attention, the
    residual adds and SwiGLU."""
    res = subprocess.run([LAYER_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-5000:], res.stderr[-1000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "SKIP" not in res.stdout.split("GPU:")[1], "the accelerator half did not run"
    for line in ("GPU: same hidden states", "GPU and CPU agree", "OK (0 failures)"):
        assert line in res.stdout
    assert "FAIL" not in res.stdout


ATTN_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_attention_hip")


@pytest.mark.gpu
@needs_ref_program(ATTN_EXE)
def test_reference_own_attention_test_passes_on_this_backend():
    """The reference's tests/test_attention.c, unmodified: prefill attention at
    28 query / 4 KV heads of 128 against its FP64 reference, at lengths on and
    off every tile boundary, with and without the chunked-prefill offset
    (bars: max |err| < 4e-3, cosine > 0.9999), then its timing loop."""
    res = subprocess.run([ATTN_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-5000:], res.stderr[-1000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "FAIL" not in res.stdout and "SKIP" not in res.stdout
    assert res.stdout.count("  ok  ") >= 8


POOL_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_kv_pool_hip")


@pytest.mark.gpu
@needs_ref_program(POOL_EXE)
def test_reference_own_kv_pool_test_passes_on_this_backend():
    """The reference's tests/test_kv_pool.c with the reference's KV cache code:
    the paged pool's bookkeeping against the device page table this backend
    writes (vv_kv_page_map_dev), exhaustion, and four threads contending."""
    res = subprocess.run([POOL_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "PASS" in res.stdout and "FAIL" not in res.stdout and "SKIP" not in res.stdout


INT8_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_int8_linear_hip")


@pytest.mark.gpu
@needs_ref_program(INT8_EXE)
def test_reference_own_int8_linear_test_passes_on_this_backend():
    """The reference's tests/test_int8_linear.c: its CPU quantiser and linear
    kernels, then this backend's activation quantisers (plain and fused, four
    orders, bit for bit against the CPU quantiser), column absmax, and the W8A8
    / W4A8 linear layers on every kernel family (exact integers with unit
    scales, FP16 outputs with bias and an aliased residual, shared-input
    launches)."""
    res = subprocess.run([INT8_EXE], capture_output=True, text=True, timeout=280)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "FAIL" not in res.stdout and "SKIPPED" not in res.stdout
    last = res.stdout.strip().splitlines()[-1]
    done, total = last.strip("= ").split()[0].split("/")
    assert done == total and int(total) >= 1600, last


W4A16_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_w4a16_hip")


@pytest.mark.gpu
@needs_ref_program(W4A16_EXE)
def test_reference_own_w4a16_test_passes_on_this_backend():
    """The reference's tests/test_w4a16.c: AWQ, GPTQ (symmetric, act-order) and
    load-time INT4 weights made and repacked by the reference's host code, then
    this backend's GEMV, fused GEMV, gather and GEMM at ten row counts against
    the reference's CPU kernel and an FP64 product of the exact FP16 weights."""
    res = subprocess.run([W4A16_EXE], capture_output=True, text=True, timeout=580)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "FAIL" not in res.stdout and "SKIP" not in res.stdout
    assert "all W4A16 checks match the reference" in res.stdout


KVQ_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_kv_quant_hip")
POS_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_decode_position_hip")


@pytest.mark.gpu
@needs_ref_program(KVQ_EXE)
def test_reference_own_kv_quant_test_passes_on_this_backend():
    """The reference's tests/test_kv_quant.c: a cache shaped like Qwen2's keys
    stored in both FP8 and all four TurboQuant formats, unpacked, attended to
    (rotating Q and un-rotating the output where the format asks), and compared
    with FP16 attention by cosine against the reference's own bars."""
    res = subprocess.run([KVQ_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "PASSED" in res.stdout and "FAIL" not in res.stdout and "SKIP" not in res.stdout
    assert res.stdout.count(" ok") >= 7


@pytest.mark.gpu
@needs_ref_program(POS_EXE)
def test_reference_own_decode_position_test_passes_on_this_backend():
    """The reference's tests/test_decode_position.c: everything a captured decode
    step reads from a device int (position add, the row copy, FP16 and
    TurboQuant decode and store, RoPE) must give the bytes the host value gives,
    and the decode launch shape must hold across a 1024-position bucket."""
    res = subprocess.run([POS_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "FAIL" not in res.stdout and "SKIP" not in res.stdout
    assert res.stdout.count("  ok  ") >= 14


ATTN_BACKENDS_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_attn_backends_hip")
CONCURRENT_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_concurrent_decode_hip")


@pytest.mark.gpu
@needs_ref_program(ATTN_BACKENDS_EXE)
def test_reference_own_attention_interface_test_passes_on_this_backend():
    """The reference's tests/test_attn_backends.c: every backend name over slab
    and paged caches in FP16, FP8 and TurboQuant, prefill and decode at two head
    layouts, against a CPU attention over the cache as vv_kv_dequant_dev returns
    it (so that call must hand back original-space vectors), and paged against
    contiguous on shuffled pages."""
    res = subprocess.run([ATTN_BACKENDS_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "every backend matches the reference" in res.stdout
    assert "FAIL" not in res.stdout and "SKIP" not in res.stdout
    assert res.stdout.count("  ok ") >= 300


@pytest.mark.gpu
@needs_ref_program(CONCURRENT_EXE)
def test_reference_own_concurrent_decode_test_passes_on_this_backend():
    """The reference's tests/test_concurrent_decode.c: four threads, each with
    its own stream and scratch, decode over slab caches and over pages of one
    shared pool; every answer must equal the single-threaded one."""
    res = subprocess.run([CONCURRENT_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "PASS" in res.stdout and "FAIL" not in res.stdout and "SKIP" not in res.stdout


SKINNY_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_skinny_hip")


@pytest.mark.gpu
@needs_ref_program(SKINNY_EXE)
def test_reference_own_small_m_test_passes_on_this_backend():
    """The reference's tests/test_skinny.c: dense FP16, per-channel INT8 and NF4
    linear layers at every row count where a tiling changes between 9 and 64,
    the small-M entry point against dequantise + vv_gemm_fp16_tile_dev +
    vv_bias_add_dev byte for byte, the public GEMM entry points likewise, all
    against its CPU kernels and an FP64 bound; q/k/v and gate/up in one launch
    against separate launches; the shapes a backend must decline."""
    res = subprocess.run([SKINNY_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "match the tile path byte for byte" in res.stdout
    assert "FAIL" not in res.stdout and "SKIP" not in res.stdout
    assert res.stdout.count("  ok  ") >= 250


BITNET_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_bitnet_hip")


@pytest.mark.gpu
@pytest.mark.skip(reason="BitNet's requantiser and int8 tied head are not built in this backend (removed: they followed the "
                         "reference's CUDA kernels too closely, and the component is outside the layer-kernel scope), and "
                         "the reference's program needs them")
def test_reference_own_bitnet_test_passes_on_this_backend():
    """The reference's tests/test_bitnet.c: its CPU integer kernels on every ISA
    the host offers against scalar references, then the accelerator's quantiser,
    ternary and int8 products, requantisation and int8 head against the CPU,
    all with ==."""
    res = subprocess.run([BITNET_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:]
    assert "FAIL" not in res.stdout


VAE_EXE = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "test_vae_stream_hip")


@pytest.mark.gpu
@pytest.mark.skip(reason="the Conv-VAE convolutions, context copy and 1/rms are not built in this backend (removed: they "
                         "followed the reference's CUDA kernels too closely, and the component is outside the "
                         "layer-kernel scope), and the reference's program needs them")
def test_reference_own_vae_stream_test_passes_on_this_backend():
    """The reference's tests/test_vae_stream.c: its whole Conv-VAE host pipeline
    (encoder plan, streaming state, front end, speech connectors) on a tiny
    random-weight model, driving this backend's kernels: against its FP32 and
    CPU encoders, batched == one by one, any chunking == the whole signal,
    conv-as-GEMM == direct conv and every GEMM tile == every other, bit for bit,
    four threads at once == alone."""
    res = subprocess.run([VAE_EXE], capture_output=True, text=True, timeout=110)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-2000:]
    assert "FAIL" not in res.stdout and "FAIL" not in res.stderr and "SKIP" not in res.stdout
    assert "43/43 passed" in res.stdout
