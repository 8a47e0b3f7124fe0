#!/usr/bin/env python3
"""Benchmark of the fused layer kernels at the Qwen2-7B prefill shape.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-layer] [--only NAME]

One "step" is one pass of the hot path over a T = 14449 token prompt:
  gather+norm   vv_embedding_rmsnorm_dev   table [152064,3584] -> hidden, normed
  add+norm      vv_add_rmsnorm_dev         residual, x [T,3584] -> residual, normed
  rope          vv_rope_qk_dev             Q [T,28,128], K [T,4,128] in place
  swiglu        vv_swiglu_dev              gate, up [T,18944] -> out
All inputs are resident in HBM before the timed region. Buffers rotate over
several distinct sets so that no launch finds its data in the last-level cache
left by the previous one. Reported:
  value      algorithmic bytes of one step / wall time of one step (GB/s), K steps
             timed between device synchronisations;
  kernels    per kernel: HIP-event time of back-to-back launches, GB/s on the
             algorithmic byte count, rows/s, fraction of the 8 TB/s HBM peak;
  roofline   the dominant kernel (SwiGLU: 63 % of the step's bytes);
  cpu_baseline  the reference's CPU kernels (or our restatement of them) on the
             host's cores, on the same T = 14449 step (about 10 s including input generation);
  configs    the reference's own launch shapes (512-4096 rows), cold;
  layer      the FP16 GEMM and attention entry points at the layer's shapes (not part of
             `value`; --no-layer skips them, --layer / --layer-fp16 add the quantised and
             whole-token legs).
Prints one JSON line on stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

T_FULL, H, I_FF, V, NQ, NK, HD = 14449, 3584, 18944, 152064, 28, 4, 128
EPS, THETA = 1e-6, 1e6
HBM_PEAK_GBPS = 8000.0           # MI355X HBM3E, published peak
CPU_SAMPLE_ROWS = T_FULL         # the whole step: ~0.3 s per pass on 8-16 host cores


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_bytes(T: int) -> dict:
    """FP16 I/O bytes each kernel must move, per launch."""
    return {
        "gather+norm": 6 * T * H + 4 * T + 2 * H,      # read row + id, write hidden + normed
        "add+norm": 8 * T * H + 2 * H,                 # read x, residual; write residual, normed
        "rope": 4 * T * (NQ + NK) * HD,                # read + write Q and K
        "swiglu": 6 * T * I_FF,                        # read gate, up; write out
        # unfused reference-API forms, timed only with --unfused (not part of the step)
        "embedding": T * (4 + 4 * H),
        "rmsnorm": 4 * T * H + 2 * H,
        "residual_add": 6 * T * H,
        "rope_q": 4 * T * NQ * HD,
        "rope_k": 4 * T * NK * HD,
        # int8-activation fused forms: FP16 in, int8 + scale + per-32 sums out
        "act_quant": 2 * T * H + T * H + 4 * T + T * H // 8,
        "rmsnorm_q8": 2 * T * H + 2 * H + T * H + 4 * T + T * H // 8,
        "swiglu_q8": 4 * T * I_FF + T * I_FF + 4 * T + T * I_FF // 8,
    }


class Workload:
    """Device buffers for `nsets` rotating copies of the step's tensors."""

    def __init__(self, torch, dev, T: int, nsets: int, table=None, weight=None):
        self.torch, self.dev, self.T, self.nsets = torch, dev, T, nsets
        gen = torch.Generator(device="cuda").manual_seed(0)

        def randn(*shape, std=1.0, mean=0.0):
            return (torch.randn(*shape, generator=gen, device="cuda") * std + mean).half()

        self.table = table if table is not None else randn(V, H, std=0.02)
        self.weight = weight if weight is not None else randn(H, std=0.1, mean=1.0)
        self.sets = []
        for s in range(nsets):
            d = {
                "ids": torch.randint(0, V, (T,), generator=gen, device="cuda", dtype=torch.int32),
                "hidden": torch.empty(T, H, dtype=torch.float16, device="cuda"),
                "normed": torch.empty(T, H, dtype=torch.float16, device="cuda"),
                "residual": randn(T, H),
                "x": randn(T, H),
                "q": randn(T, NQ, HD),
                "k": randn(T, NK, HD),
                "gate": randn(T, I_FF, std=2.0),
                "up": randn(T, I_FF, std=2.0),
                "out": torch.empty(T, I_FF, dtype=torch.float16, device="cuda"),
            }
            self.sets.append(d)
        torch.cuda.synchronize()

    def q8_buffers(self):
        if not hasattr(self, "_q8"):
            t = self.torch
            self._q8 = (t.empty(self.T * I_FF, dtype=t.int8, device="cuda"),
                        t.empty(self.T, dtype=t.float32, device="cuda"),
                        t.empty(self.T * I_FF // 32, dtype=t.int32, device="cuda"))
        return self._q8

    def launch(self, name: str, i: int, st: int) -> None:
        d, dev, T = self.sets[i % self.nsets], self.dev, self.T
        if name == "gather+norm":
            rc = dev.vv_embedding_rmsnorm_dev(self.table.data_ptr(), d["ids"].data_ptr(),
                                              self.weight.data_ptr(), d["hidden"].data_ptr(),
                                              d["normed"].data_ptr(), T, H, EPS, st)
        elif name == "add+norm":
            rc = dev.vv_add_rmsnorm_dev(d["residual"].data_ptr(), d["x"].data_ptr(),
                                        self.weight.data_ptr(), d["normed"].data_ptr(),
                                        T, H, EPS, st)
        elif name == "rope":
            rc = dev.vv_rope_qk_dev(d["q"].data_ptr(), d["k"].data_ptr(), T, NQ, NK, HD, 0, None,
                                    THETA, st)
        elif name == "swiglu":
            rc = dev.vv_swiglu_dev(d["gate"].data_ptr(), d["up"].data_ptr(), d["out"].data_ptr(),
                                   T * I_FF, st)
        elif name == "embedding":
            rc = dev.vv_embedding_dev(self.table.data_ptr(), d["ids"].data_ptr(),
                                      d["hidden"].data_ptr(), T, H, st)
        elif name == "rmsnorm":
            rc = dev.vv_rmsnorm_dev(d["x"].data_ptr(), self.weight.data_ptr(),
                                    d["normed"].data_ptr(), T, H, EPS, st)
        elif name == "residual_add":
            rc = dev.vv_residual_add_dev(d["residual"].data_ptr(), d["x"].data_ptr(), T * H, st)
        elif name == "act_quant":
            q = self.q8_buffers()
            rc = dev.vv_act_quant_dev(d["x"].data_ptr(), T, H, 0, q[0].data_ptr(), q[1].data_ptr(),
                                      q[2].data_ptr(), st)
        elif name == "rmsnorm_q8":
            q = self.q8_buffers()
            rc = dev.vv_rmsnorm_q8_dev(d["x"].data_ptr(), self.weight.data_ptr(), T, H, EPS, 0,
                                       q[0].data_ptr(), q[1].data_ptr(), q[2].data_ptr(), st)
        elif name == "swiglu_q8":
            q = self.q8_buffers()
            rc = dev.vv_swiglu_q8_dev(d["gate"].data_ptr(), d["up"].data_ptr(), T, I_FF, 0,
                                      q[0].data_ptr(), q[1].data_ptr(), q[2].data_ptr(), st)
        elif name == "rope_q":
            rc = dev.vv_rope_dev(d["q"].data_ptr(), T, NQ, HD, 0, None, THETA, st)
        elif name == "rope_k":
            rc = dev.vv_rope_dev(d["k"].data_ptr(), T, NK, HD, 0, None, THETA, st)
        else:
            raise KeyError(name)
        if rc != 0:
            raise RuntimeError(f"{name} returned status {rc}")


KERNELS = ["gather+norm", "add+norm", "rope", "swiglu"]
UNFUSED = ["embedding", "rmsnorm", "residual_add", "rope_q", "rope_k", "act_quant", "rmsnorm_q8",
           "swiglu_q8"]


def time_kernel(torch, wl: Workload, name: str, launches: int, reps: int, st: int):
    """HIP events on the launch stream around `launches` back-to-back launches;
    returns (best, median) seconds per launch over `reps` repetitions."""
    per = []
    for _ in range(reps):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(launches):
            wl.launch(name, i, st)
        e1.record()
        e1.synchronize()
        per.append(e0.elapsed_time(e1) * 1e-3 / launches)
    per.sort()
    return per[0], per[len(per) // 2]


# The shapes BASELINE.json's configs name, and the 2048-row chunk the reference's chunked prefill
# actually launches (src/inference/decoder.c:1147-1174).
CONFIG_SHAPES = [("add+norm", 512), ("add+norm", 2048), ("add+norm", 4096), ("rope", 2048),
                 ("swiglu", 2048), ("swiglu", 4096), ("gather+norm", 2048)]
LLC_BYTES = 256 << 20            # the last-level cache in front of HBM (plus 4 MB of L2 per XCD)
CONFIG_FOOTPRINT = 4 * LLC_BYTES   # rotate over at least this many bytes of distinct tensors


def configs_leg(torch, dev, wl: "Workload", st: int, launches: int = 120, reps: int = 5) -> list:
    """Every (kernel, T) of CONFIG_SHAPES, cold: the launches rotate over enough distinct buffer
    sets that their joint footprint is four times the last-level cache, so no launch finds its
    inputs cached by an earlier one. These launches last 3-70 us, less than Python needs to issue
    one, so the stream is first kept busy by a few full-size SwiGLU launches while the timed
    launches are queued behind them; the start event sits between the two groups. The time per
    launch therefore includes the gap between dependent kernels of one stream, as in the product."""
    # What a short launch can reach on this device is measured here, not modelled: beside every config the same
    # number of bytes (half read, half written) goes through the library's plain copy kernel (vv_dev_memcpy_d2d)
    # under the same conditions - cold rotating buffers, queued behind the same work - and a one-row launch of
    # the same entry point gives the cost of a launch that moves nothing.
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    wl1 = Workload(torch, dev, 1, 1, table=wl.table, weight=wl.weight)
    floors = {}
    for name in KERNELS:
        for i in range(8):
            wl.launch("swiglu", i, st)
        e0.record()
        for i in range(200):
            wl1.launch(name, i, st)
        e1.record()
        e1.synchronize()
        floors[name] = e0.elapsed_time(e1) * 1e-3 / 200
    log("  one-row launches, queued: " + ", ".join(f"{k} {v * 1e6:.2f} us" for k, v in floors.items()))
    out = []
    for name, T in CONFIG_SHAPES:
        nbytes = algorithmic_bytes(T)[name]
        nsets = max(3, -(-CONFIG_FOOTPRINT // nbytes))
        gen = torch.Generator(device="cuda").manual_seed(T)

        def randn(*shape, std=1.0):
            return (torch.randn(*shape, generator=gen, device="cuda") * std).half()

        sets = []
        for _ in range(nsets):
            if name == "add+norm":
                d = {"residual": randn(T, H), "x": randn(T, H),
                     "normed": torch.empty(T, H, dtype=torch.float16, device="cuda")}
            elif name == "rope":
                d = {"q": randn(T, NQ, HD), "k": randn(T, NK, HD)}
            elif name == "swiglu":
                d = {"gate": randn(T, I_FF, std=2.0), "up": randn(T, I_FF, std=2.0),
                     "out": torch.empty(T, I_FF, dtype=torch.float16, device="cuda")}
            else:
                d = {"ids": torch.randint(0, V, (T,), generator=gen, device="cuda", dtype=torch.int32),
                     "hidden": torch.empty(T, H, dtype=torch.float16, device="cuda"),
                     "normed": torch.empty(T, H, dtype=torch.float16, device="cuda")}
            sets.append(d)
        small = Workload.__new__(Workload)
        small.torch, small.dev, small.T, small.nsets = torch, dev, T, nsets
        small.table, small.weight, small.sets = wl.table, wl.weight, sets
        n = max(launches, 2 * nsets)
        for i in range(nsets):
            small.launch(name, i, st)
        torch.cuda.synchronize()
        per, queued_ahead = [], True
        for _ in range(reps):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            for i in range(8):                      # ~2 ms of work ahead of the timed launches
                wl.launch("swiglu", i, st)
            e0.record()
            for i in range(n):
                small.launch(name, i, st)
            e1.record()
            queued_ahead = queued_ahead and not e0.query()     # still busy ahead of us: the queue never ran dry
            e1.synchronize()
            per.append(e0.elapsed_time(e1) * 1e-3 / n)
        per.sort()
        med = per[len(per) // 2]
        # the plain copy of the same bytes, timed the same way
        del sets, small
        torch.cuda.empty_cache()
        half = (nbytes // 2 + 15) // 16 * 16
        pairs = [(torch.empty(half, dtype=torch.uint8, device="cuda"), torch.empty(half, dtype=torch.uint8, device="cuda"))
                 for _ in range(nsets)]
        for a, b in pairs:
            a.zero_()
            dev.vv_dev_memcpy_d2d(b.data_ptr(), a.data_ptr(), half, st)
        torch.cuda.synchronize()
        cper = []
        for _ in range(reps):
            for i in range(8):
                wl.launch("swiglu", i, st)
            e0.record()
            for i in range(n):
                a, b = pairs[i % nsets]
                dev.vv_dev_memcpy_d2d(b.data_ptr(), a.data_ptr(), half, st)
            e1.record()
            e1.synchronize()
            cper.append(e0.elapsed_time(e1) * 1e-3 / n)
        cper.sort()
        copy_s = cper[len(cper) // 2]
        del pairs
        out.append({"kernel": name, "rows": T, "bytes": nbytes, "us": med * 1e6, "us_best": per[0] * 1e6,
                    "GBps": nbytes / med / 1e9, "frac": nbytes / med / 1e9 / HBM_PEAK_GBPS,
                    "rows_per_s": T / med, "buffer_sets": nsets, "footprint_MB": nsets * nbytes / 1e6,
                    "cold": True, "launches_queued_ahead_of_the_gpu": bool(queued_ahead),
                    "floor_us": floors[name] * 1e6, "plain_copy_of_the_same_bytes_us": copy_s * 1e6,
                    "plain_copy_frac": 2.0 * half / copy_s / 1e9 / HBM_PEAK_GBPS})
        log(f"  config {name:12s} T={T:5d} {med * 1e6:8.2f} us  {nbytes / med / 1e9:8.1f} GB/s  "
            f"{100 * nbytes / med / 1e9 / HBM_PEAK_GBPS:5.1f} % of peak  ({nsets} sets, cold"
            f"{'' if queued_ahead else ', issue-bound'}; a plain copy of the same bytes: {copy_s * 1e6:.2f} us = "
            f"{100 * out[-1]['plain_copy_frac']:.1f} %)")
        torch.cuda.empty_cache()
    return out


def decode_graph_leg(torch, dev, wl1) -> dict:
    """One token's worth of this library's launches (per layer: norm -> RoPE(Q,K) with the
    position read from device memory -> add+norm -> SwiGLU -> add+norm), issued directly and
    as a captured graph replayed; the position advances inside the graph (vv_pos_add_dev)."""
    import ctypes as C
    d = wl1.sets[0]
    w = wl1.weight.data_ptr()
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    s = C.c_void_p()
    assert dev.vv_dev_stream_create(C.byref(s)) == 0
    st = s.value
    layers = 28

    def issue():
        n = 0
        for _ in range(layers):
            assert dev.vv_rmsnorm_dev(d["hidden"].data_ptr(), w, d["normed"].data_ptr(), 1, H, EPS, st) == 0
            assert dev.vv_rope_qk_dev(d["q"].data_ptr(), d["k"].data_ptr(), 1, NQ, NK, HD, 0,
                                      pos.data_ptr(), THETA, st) == 0
            assert dev.vv_add_rmsnorm_dev(d["residual"].data_ptr(), d["x"].data_ptr(), w,
                                          d["normed"].data_ptr(), 1, H, EPS, st) == 0
            assert dev.vv_swiglu_dev(d["gate"].data_ptr(), d["up"].data_ptr(), d["gate"].data_ptr(),
                                     I_FF, st) == 0
            assert dev.vv_add_rmsnorm_dev(d["residual"].data_ptr(), d["x"].data_ptr(), w,
                                          d["normed"].data_ptr(), 1, H, EPS, st) == 0
            n += 5
        assert dev.vv_pos_add_dev(pos.data_ptr(), pos.data_ptr(), 1, st) == 0
        return n + 1

    torch.cuda.synchronize()
    launches = issue()
    assert dev.vv_dev_stream_sync(st) == 0
    reps = 20
    t0 = time.perf_counter()
    for _ in range(reps):
        issue()
    assert dev.vv_dev_stream_sync(st) == 0
    eager = (time.perf_counter() - t0) / reps
    assert dev.vv_dev_graph_begin(st) == 0
    issue()
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(st, C.byref(g)) == 0 and g.value
    for _ in range(3):
        assert dev.vv_dev_graph_launch(g.value, st) == 0
    assert dev.vv_dev_stream_sync(st) == 0
    before = int(pos.item())
    t0 = time.perf_counter()
    for _ in range(reps):
        assert dev.vv_dev_graph_launch(g.value, st) == 0
    assert dev.vv_dev_stream_sync(st) == 0
    replay = (time.perf_counter() - t0) / reps
    assert int(pos.item()) == before + reps          # every replay advanced the device-side position
    dev.vv_dev_graph_destroy(g.value)
    dev.vv_dev_stream_destroy(st)
    return {"launches": launches, "eager_us": eager * 1e6, "replay_us": replay * 1e6,
            "replay_us_per_launch": replay * 1e6 / launches}


MFMA_F16_PEAK_TFLOPS = 2500.0        # MI355X dense FP16 matrix rate
MFMA_I8_PEAK_TOPS = 5000.0           # and the dense int8 one


def layer_leg(torch, dev, T: int, st: int, fp16_only: bool = False) -> dict:
    """The rest of a dense Qwen2-7B layer at the same prompt length: the four projection shapes of
    the FP16 GEMM and causal GQA attention at M = T (matrix-core bound: TFLOP/s against the dense
    FP16 peak), and the decode forms (one row: bound by the weight / cache bytes, GB/s). Not part of
    the step; the causal FLOP count is 4 * heads * head_dim * T(T+1)/2."""
    import ctypes as C

    def timed(fn, launches, reps=3):
        fn()
        per = []
        for _ in range(reps):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(launches):
                fn()
            e1.record()
            e1.synchronize()
            per.append(e0.elapsed_time(e1) * 1e-3 / launches)
        per.sort()
        return per[len(per) // 2]

    # "gemm_chunk": the same projections at 2048 rows, the reference's prefill chunk (decoder.c:1147-1174)
    out = {"gemm": {}, "gemm_chunk": {}, "gemv": {}}
    shapes = (("q_o_proj", H, H), ("kv_proj", NK * HD, H), ("gate_up_proj", I_FF, H), ("down_proj", H, I_FF))
    for name, n, k in shapes:
        w = torch.randn(n, k, dtype=torch.float16, device="cuda") * k ** -0.5
        for m, key in ((T, "gemm"), (2048, "gemm_chunk"), (1, "gemv")):
            a = torch.randn(m, k, dtype=torch.float16, device="cuda")
            c = torch.empty(m, n, dtype=torch.float16, device="cuda")
            sec = timed(lambda: dev.vv_gemm_fp16_dev(a.data_ptr(), w.data_ptr(), c.data_ptr(), m, n, k,
                                                     1.0, 0.0, st), 5 if m > 1 else 50)
            if m > 1:
                tf = 2.0 * m * n * k / sec / 1e12
                out[key][name] = {"M": m, "N": n, "K": k, "us": sec * 1e6, "TFLOPs": tf,
                                  "frac_of_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS}
            else:
                gb = 2.0 * (n * k + k + n) / sec / 1e9
                out[key][name] = {"N": n, "K": k, "us": sec * 1e6, "GBps": gb,
                                  "frac_of_hbm_peak": gb / HBM_PEAK_GBPS}
            del a, c
        del w
    # gate, up and SwiGLU in one GEMM (vv_gemm_swiglu_dev) against the three launches it replaces
    out["gemm_swiglu"] = {}
    wg = torch.randn(I_FF, H, dtype=torch.float16, device="cuda") * H ** -0.5
    wu = torch.randn(I_FF, H, dtype=torch.float16, device="cuda") * H ** -0.5
    for m in (T, 2048):
        a = torch.randn(m, H, dtype=torch.float16, device="cuda")
        g, u = (torch.empty(m, I_FF, dtype=torch.float16, device="cuda") for _ in range(2))

        def three():
            dev.vv_gemm_fp16_dev(a.data_ptr(), wg.data_ptr(), g.data_ptr(), m, I_FF, H, 1.0, 0.0, st)
            dev.vv_gemm_fp16_dev(a.data_ptr(), wu.data_ptr(), u.data_ptr(), m, I_FF, H, 1.0, 0.0, st)
            dev.vv_swiglu_dev(g.data_ptr(), u.data_ptr(), g.data_ptr(), m * I_FF, st)
        sec = timed(lambda: dev.vv_gemm_swiglu_dev(a.data_ptr(), wg.data_ptr(), wu.data_ptr(), None, None,
                                                   g.data_ptr(), m, I_FF, H, st), 5)
        sec3 = timed(three, 5)
        tf = 4.0 * m * I_FF * H / sec / 1e12
        out["gemm_swiglu"][f"M{m}"] = {"M": m, "N": I_FF, "K": H, "us": sec * 1e6, "TFLOPs": tf,
                                       "frac_of_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS,
                                       "us_two_gemms_and_swiglu": sec3 * 1e6}
        del a, g, u
    del wg, wu
    if not fp16_only:
        # The same four projections as W8A8 (int8 x int8 on the matrix cores, per-row / per-channel scales).
        out["w8a8"], out["w8a8_gemv"] = {}, {}
        for name, n, k in shapes:
            w8 = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda")
            sw = torch.rand(n, dtype=torch.float32, device="cuda") * 1e-2
            for m, key in ((T, "w8a8"), (1, "w8a8_gemv")):
                xq = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda")
                sx = torch.rand(m, dtype=torch.float32, device="cuda") * 1e-2
                c = torch.empty(m, n, dtype=torch.float16, device="cuda")
                sec = timed(lambda: dev.vv_w8a8_linear_dev(xq.data_ptr(), sx.data_ptr(), w8.data_ptr(), sw.data_ptr(),
                                                           None, None, c.data_ptr(), 0, m, n, k, 0, st),
                            5 if m > 1 else 50)
                if m > 1:
                    tops = 2.0 * m * n * k / sec / 1e12
                    out[key][name] = {"M": m, "N": n, "K": k, "us": sec * 1e6, "TOPs": tops,
                                      "frac_of_mfma_peak": tops / MFMA_I8_PEAK_TOPS}
                else:
                    gb = (n * k + k + 6.0 * n) / sec / 1e9
                    out[key][name] = {"N": n, "K": k, "us": sec * 1e6, "GBps": gb,
                                      "frac_of_hbm_peak": gb / HBM_PEAK_GBPS}
                del xq, sx, c
            del w8, sw
        # And as W4A8: 4-bit codes with a scale and a zero point per 128 columns (any bytes are valid codes).
        out["w4a8"], out["w4a8_gemv"], out["w4a8_chunk"] = {}, {}, {}
        G = 128
        for name, n, k in shapes:
            w4 = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda")
            sz = torch.stack([torch.rand(n, k // G, device="cuda") * 0.02 + 0.002,
                              torch.randint(0, 16, (n, k // G), device="cuda").float()], dim=-1).half().contiguous()
            # T rows (prefill), one row (decode) and 29 rows (a streaming chunk: the weights are still the bytes)
            for m, key, layout in ((T, "w4a8", 3), (1, "w4a8_gemv", 2), (29, "w4a8_chunk", 3)):
                xq = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda")
                sx = torch.rand(m, dtype=torch.float32, device="cuda") * 1e-2
                c = torch.empty(m, n, dtype=torch.float16, device="cuda")
                xs = xq.view(m, k // 32, 32).sum(-1, dtype=torch.int32).contiguous()     # what the quantiser writes
                sec = timed(lambda: dev.vv_w4a8_linear_dev(xq.data_ptr(), layout, sx.data_ptr(), xs.data_ptr(), w4.data_ptr(),
                                                           sz.data_ptr(), G, None, None, c.data_ptr(), 0, m, n, k, 0,
                                                           st), 5 if m > 64 else 50)
                if m > 64:
                    tops = 2.0 * m * n * k / sec / 1e12
                    out[key][name] = {"M": m, "N": n, "K": k, "group": G, "us": sec * 1e6, "TOPs": tops,
                                      "frac_of_mfma_peak": tops / MFMA_I8_PEAK_TOPS}
                else:
                    gb = (n * k / 2 + n * (k // G) * 4 + m * (k + 2.0 * n)) / sec / 1e9
                    out[key][name] = {"M": m, "N": n, "K": k, "group": G, "us": sec * 1e6, "GBps": gb,
                                      "frac_of_hbm_peak": gb / HBM_PEAK_GBPS}
                del xq, sx, c
            # the same codes against FP16 activations (W4A16)
            for m, key in ((T, "w4a16"), (1, "w4a16_gemv"), (29, "w4a16_chunk")):
                out.setdefault(key, {})
                a = torch.randn(m, k, dtype=torch.float16, device="cuda")
                c = torch.empty(m, n, dtype=torch.float16, device="cuda")
                dense = torch.empty(n * k, dtype=torch.float16, device="cuda")     # the decoder's dequant scratch
                sec = timed(lambda: dev.vv_w4a16_gemm_dev(a.data_ptr(), w4.data_ptr(), sz.data_ptr(), None, c.data_ptr(),
                                                          dense.data_ptr(), n * k * 2, m, n, k, G, st),
                            5 if m > 64 else 50)
                if m > 64:
                    tf = 2.0 * m * n * k / sec / 1e12
                    out[key][name] = {"M": m, "N": n, "K": k, "group": G, "us": sec * 1e6, "TFLOPs": tf,
                                      "frac_of_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS}
                else:
                    gb = (n * k / 2 + n * (k // G) * 4 + m * (2.0 * k + 2.0 * n)) / sec / 1e9
                    out[key][name] = {"M": m, "N": n, "K": k, "group": G, "us": sec * 1e6, "GBps": gb,
                                      "frac_of_hbm_peak": gb / HBM_PEAK_GBPS}
                del a, c, dense
            del w4, sz
        # The older weight-only formats on FP16 activations: one row (decode), 29 rows (a streaming
        # chunk, the small-M kernel where it serves) and the dequantiser that feeds the FP16 GEMM.
        out["weight_only"] = {}
        for fmt in ("int8", "nf4", "int4"):
            for name, n, k in shapes:
                if fmt == "int8":
                    wq = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda")
                    sc = torch.rand(n, dtype=torch.float32, device="cuda") * 1e-2
                    mn, wbytes = None, n * k + 4.0 * n
                else:
                    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda")
                    per = 64 if fmt == "nf4" else G
                    sc = (torch.rand(n * k // per, device="cuda") * 0.02 + 0.002).half()
                    mn = (-torch.rand(n * k // per, device="cuda") * 0.1).half() if fmt == "int4" else None
                    wbytes = n * k / 2 + (2.0 if fmt == "nf4" else 4.0) * n * k / per
                dense = torch.empty(n * k, dtype=torch.float16, device="cuda")
                P = lambda t: t.data_ptr() if t is not None else None

                def run(m, a, c):
                    if fmt == "int8":
                        return dev.vv_int8_gemm_dev(P(a), P(wq), P(sc), P(c), P(dense), m, n, k, st)
                    if fmt == "nf4":
                        return dev.vv_nf4_gemm_dev(P(a), P(wq), P(sc), P(c), P(dense), m, n, k, 64, st)
                    return dev.vv_awq_gemm_dev(P(a), P(wq), P(mn), P(sc), P(c), P(dense), m, n, k, G, st)

                def run_dequant():
                    if fmt == "int8":
                        return dev.vv_dequant_int8_dev(P(wq), P(sc), P(dense), n, k, st)
                    if fmt == "nf4":
                        return dev.vv_dequant_nf4_dev(P(wq), P(sc), P(dense), n * k, 64, st)
                    return dev.vv_dequant_awq_dev(P(wq), P(mn), P(sc), P(dense), n, k, G, st)

                d = {"N": n, "K": k}
                for m in (1, 29):
                    a = torch.randn(m, k, dtype=torch.float16, device="cuda")
                    c = torch.empty(m, n, dtype=torch.float16, device="cuda")
                    assert run(m, a, c) == 0
                    sec = timed(lambda: run(m, a, c), 50)
                    d[f"M{m}_us"] = sec * 1e6
                    if m == 1:
                        d["M1_GBps"] = (wbytes + 2.0 * k + 2.0 * n) / sec / 1e9
                        d["M1_frac_of_hbm_peak"] = d["M1_GBps"] / HBM_PEAK_GBPS
                    del a, c
                assert run_dequant() == 0
                sec = timed(run_dequant, 20)
                d["dequant_us"] = sec * 1e6
                d["dequant_GBps"] = (wbytes + 2.0 * n * k) / sec / 1e9
                out["weight_only"][f"{fmt} {name}"] = d
                del wq, sc, mn, dense
    q = torch.randn(T, NQ, HD, dtype=torch.float16, device="cuda")
    k_ = torch.randn(T, NK, HD, dtype=torch.float16, device="cuda")
    v_ = torch.randn(T, NK, HD, dtype=torch.float16, device="cuda")
    o = torch.empty_like(q)
    view = dev.KvView(k=k_.data_ptr(), v=v_.data_ptr(), k_meta=None, v_meta=None, page_table=None,
                      format=0, n_kv_heads=NK, head_dim=HD)
    sec = timed(lambda: dev.vv_attn_prefill(2, q.data_ptr(), C.addressof(view), o.data_ptr(), NQ, T, 0, T,
                                            True, None, st), 3)
    tf = 4.0 * NQ * HD * T * (T + 1) / 2 / sec / 1e12
    out["attn_prefill"] = {"rows": T, "us": sec * 1e6, "TFLOPs": tf,
                           "frac_of_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS}
    # The product's launch shape: the prompt's last 2048-row chunk (decoder.c:1147-1174) against the whole cache.
    if T > 2048:
        rows, off = 2048, T - 2048
        sec = timed(lambda: dev.vv_attn_prefill(2, q.data_ptr(), C.addressof(view), o.data_ptr(), NQ, rows, off, T,
                                                True, None, st), 5)
        tf = 4.0 * NQ * HD * (rows * off + rows * (rows + 1) / 2) / sec / 1e12
        out["attn_prefill_chunk"] = {"rows": rows, "q_offset": off, "kv_len": T, "us": sec * 1e6, "TFLOPs": tf,
                                     "frac_of_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS}
    scratch = torch.empty(dev.vv_attn_scratch_bytes(NQ, NK, HD), dtype=torch.uint8, device="cuda")
    # Decode reads each layer's cache once per token: 28 caches in rotation (829 MB at T = 14449, so nothing
    # is served from the last-level cache), issued one by one and as one captured graph replayed.
    caches = [(torch.randn(T, NK, HD, dtype=torch.float16, device="cuda"),
               torch.randn(T, NK, HD, dtype=torch.float16, device="cuda")) for _ in range(28)]
    views = [dev.KvView(k=kk.data_ptr(), v=vv.data_ptr(), k_meta=None, v_meta=None, page_table=None,
                        format=0, n_kv_heads=NK, head_dim=HD) for kk, vv in caches]

    ds = C.c_void_p()                      # a stream of its own: the default stream cannot be captured
    assert dev.vv_dev_stream_create(C.byref(ds)) == 0

    def decode_all():
        for vw in views:
            assert dev.vv_attn_decode(2, q.data_ptr(), C.addressof(vw), o.data_ptr(), NQ, T, None,
                                      scratch.data_ptr(), ds.value) == 0

    def wall(fn, reps=10):                 # host clock around a drained stream, median of three
        fn()
        assert dev.vv_dev_stream_sync(ds.value) == 0
        per = []
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(reps):
                fn()
            assert dev.vv_dev_stream_sync(ds.value) == 0
            per.append((time.perf_counter() - t0) / reps)
        return sorted(per)[1]

    torch.cuda.synchronize()
    sec = wall(decode_all) / len(views)
    assert dev.vv_dev_graph_begin(ds.value) == 0
    decode_all()
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(ds.value, C.byref(g)) == 0 and g.value
    sec_graph = wall(lambda: dev.vv_dev_graph_launch(g.value, ds.value)) / len(views)
    dev.vv_dev_graph_destroy(g.value)
    dev.vv_dev_stream_destroy(ds.value)
    nbytes = 2.0 * T * NK * HD * 2
    out["attn_decode"] = {"cache_len": T, "caches_in_rotation": len(views), "us": sec * 1e6, "GBps": nbytes / sec / 1e9,
                          "frac_of_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS, "graph_us": sec_graph * 1e6,
                          "graph_GBps": nbytes / sec_graph / 1e9,
                          "note": "two launches per call (slices, then their merge); about 8 us of it is launch and "
                                  "memory latency, the same at 1000 positions"}
    del caches, views
    if not fp16_only:
        # The same two over an FP8 (E4M3) cache: half the cache bytes, widened on their way into the tile.
        k8 = torch.randint(0, 0x78, (T, NK, HD), dtype=torch.uint8, device="cuda")
        v8 = torch.randint(0, 0x78, (T, NK, HD), dtype=torch.uint8, device="cuda")
        view8 = dev.KvView(k=k8.data_ptr(), v=v8.data_ptr(), k_meta=None, v_meta=None, page_table=None,
                           format=1, n_kv_heads=NK, head_dim=HD)
        sec = timed(lambda: dev.vv_attn_prefill(2, q.data_ptr(), C.addressof(view8), o.data_ptr(), NQ, T, 0, T,
                                                True, None, st), 3)
        tf = 4.0 * NQ * HD * T * (T + 1) / 2 / sec / 1e12
        out["attn_prefill_fp8"] = {"rows": T, "us": sec * 1e6, "TFLOPs": tf, "frac_of_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS}
        sec = timed(lambda: dev.vv_attn_decode(2, q.data_ptr(), C.addressof(view8), o.data_ptr(), NQ, T, None,
                                               scratch.data_ptr(), st), 50)
        gb = 2.0 * T * NK * HD / sec / 1e9
        out["attn_decode_fp8"] = {"cache_len": T, "us": sec * 1e6, "GBps": gb, "frac_of_hbm_peak": gb / HBM_PEAK_GBPS}
        del k8, v8
    del q, k_, v_, o
    if not fp16_only:
        # BitNet's integer layers at the 1.5B shape (hidden 1536, FFN 8960, vocabulary 151936): quantise, one decode row
        # and a 512-row prefill through the ternary gate projection.
        Hb, Fb, Vb, Mb = 1536, 8960, 151936, 512
        bn = {}
        xb = torch.randn(Mb, Hb, dtype=torch.float16, device="cuda")
        qb = torch.empty(Mb, Hb, dtype=torch.int8, device="cuda")
        sb = torch.empty(Mb, dtype=torch.float32, device="cuda")
        smb = torch.empty(Mb, dtype=torch.int32, device="cuda")
        sec = timed(lambda: dev.vv_act_quant_i8_dev(xb.data_ptr(), 1, Mb, Hb, qb.data_ptr(), sb.data_ptr(), smb.data_ptr(), st), 50)
        bn["act_quant_512x1536_us"] = sec * 1e6
        codes = torch.randint(0, 3, (Fb, Hb // 4, 4), dtype=torch.uint8, device="cuda")
        codes = (codes[..., 0] << 6 | codes[..., 1] << 4 | codes[..., 2] << 2 | codes[..., 3]).contiguous()
        yb = torch.empty(Mb, Fb, dtype=torch.float16, device="cuda")
        for m in (1, Mb):
            sec = timed(lambda: dev.vv_ternary_gemm_dev(qb.data_ptr(), smb.data_ptr(), sb.data_ptr(), codes.data_ptr(), 0.02,
                                                        None, None, yb.data_ptr(), 1, m, Fb, Hb, st), 50)
            bn[f"ternary_{Fb}x{Hb}_M{m}_us"] = sec * 1e6
        # (the int8 tied head is not built in this backend: no leg)
        out["bitnet"] = bn
        del xb, qb, sb, smb, codes, yb
        # Conv-VAE encoder ops at a deep stage's shape: 512 channels, 24000 packed columns in one item.
        Cv, Tv, kv = 512, 24000, 7
        d = dev.VaeConvDesc()
        d.n, d.cap = 1, kv - 1
        d.it[0].in_len = d.it[0].out_len = Tv
        xv = torch.randn(Cv, Tv, dtype=torch.float16, device="cuda")
        xo = torch.empty_like(xv)
        rv = torch.empty(Tv, dtype=torch.float32, device="cuda")
        nwv = torch.randn(Cv, dtype=torch.float16, device="cuda")
        cwv = torch.randn(Cv, kv, dtype=torch.float16, device="cuda") * 0.3
        vae = {}
        rv.copy_(torch.rsqrt(xv.float().pow(2).mean(0) + 1e-5))     # the per-column 1/rms op is not built in this backend
        sec = timed(lambda: dev.vv_vae_mixer_dev(C.addressof(d), xv.data_ptr(), xo.data_ptr(), Tv, rv.data_ptr(), Tv,
                                                 nwv.data_ptr(), cwv.data_ptr(), None, nwv.data_ptr(), Cv, kv, st), 50)
        vae["mixer_us"] = sec * 1e6
        vae["mixer_GBps"] = 4.0 * Cv * Tv / sec / 1e9
        w1 = torch.randn(4 * Cv, Cv, dtype=torch.float16, device="cuda") * Cv ** -0.5
        hv = torch.empty(4 * Cv, Tv, dtype=torch.float16, device="cuda")
        sec = timed(lambda: dev.vv_vae_gemm_nn_dev(0, w1.data_ptr(), xv.data_ptr(), Tv, hv.data_ptr(), Tv, 4 * Cv, Cv, Tv,
                                                   None, None, rv.data_ptr(), nwv.data_ptr(), 0, st), 20)
        vae["ffn_up_gelu_us"] = sec * 1e6
        vae["ffn_up_gelu_TFLOPs"] = 2.0 * 4 * Cv * Cv * Tv / sec / 1e12
        out["vae"] = vae
    return out


def prefill_layer_leg(torch, dev, T: int, st: int) -> dict:
    """One dense decoder layer over the whole T-row prompt, in the reference decoder's op order
    (decoder.c:706-991), from its normed input to the next layer's: q/k/v GEMMs, bias + RoPE, causal
    attention over the chunk's own K/V, o GEMM, add + norm, gate/up GEMMs, SwiGLU, down GEMM, add + norm -
    once on this library's fused entry points, once on the calls of the reference's device.h alone.
    Random weights. Reports the layer time and what 28 such layers make in prompt tokens per second."""
    import ctypes as C
    f16 = dict(dtype=torch.float16, device="cuda")
    QD, KD = NQ * HD, NK * HD
    w = lambda *shape, std: torch.randn(*shape, **f16) * std
    wq, wk, wv, wo = w(QD, H, std=H ** -0.5), w(KD, H, std=H ** -0.5), w(KD, H, std=H ** -0.5), w(H, QD, std=QD ** -0.5)
    wg, wu, wd = w(I_FF, H, std=H ** -0.5), w(I_FF, H, std=H ** -0.5), w(H, I_FF, std=I_FF ** -0.5)
    bq, bk, bv = w(QD, std=0.1), w(KD, std=0.1), w(KD, std=0.1)
    n1, n2 = 1 + w(H, std=0.1), 1 + w(H, std=0.1)
    hidden, normed, proj = w(T, H, std=1.0), torch.empty(T, H, **f16), torch.empty(T, H, **f16)
    q, attn = torch.empty(T, QD, **f16), torch.empty(T, QD, **f16)
    k, v = torch.empty(T, KD, **f16), torch.empty(T, KD, **f16)
    gate, up = torch.empty(T, I_FF, **f16), torch.empty(T, I_FF, **f16)
    view = dev.KvView(k=k.data_ptr(), v=v.data_ptr(), k_meta=None, v_meta=None, page_table=None, format=0,
                      n_kv_heads=NK, head_dim=HD)
    P = lambda t: t.data_ptr()

    def gemm(x, wt, y, n, kk):
        assert dev.vv_gemm_fp16_dev(P(x), P(wt), P(y), T, n, kk, 1.0, 0.0, st) == 0

    # cos/sin of the prompt's positions: once per forward pass, shared by the 28 layers
    rope_table = torch.empty(T, HD // 2, 2, dtype=torch.float32, device="cuda")
    assert dev.vv_rope_table_dev(P(rope_table), T, HD, 0, None, THETA, st) == 0

    def layer(fused=True):
        """One layer from its normed input to the next layer's normed input. fused: this library's fused
        entry points; else only the calls of the reference's device.h, in decoder.c's order (706-991)."""
        if fused:
            # q / k / v with bias + RoPE in the store (one grid of equal tiles up to ~9000 rows, else one launch
            # per projection with bias + RoPE in the q / k stores)
            assert dev.vv_gemm_qkv_rope_dev(P(normed), P(wq), P(wk), P(wv), P(bq), P(bk), P(bv), P(q), P(k), P(v), T,
                                            NQ, NK, HD, H, P(rope_table), None, None, None, 0, None, st) == 0
        else:
            gemm(normed, wq, q, QD, H)
            gemm(normed, wk, k, KD, H)
            gemm(normed, wv, v, KD, H)
            assert dev.vv_bias_add_dev(P(q), P(bq), T, QD, st) == 0
            assert dev.vv_bias_add_dev(P(k), P(bk), T, KD, st) == 0
            assert dev.vv_bias_add_dev(P(v), P(bv), T, KD, st) == 0
            assert dev.vv_rope_dev(P(q), T, NQ, HD, 0, None, THETA, st) == 0
            assert dev.vv_rope_dev(P(k), T, NK, HD, 0, None, THETA, st) == 0
        assert dev.vv_attn_prefill(2, P(q), C.addressof(view), P(attn), NQ, T, 0, T, True, None, st) == 0
        gemm(attn, wo, proj, H, QD)
        if fused:
            assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n2), P(normed), T, H, EPS, st) == 0
            # gate, up and SwiGLU in one GEMM: gate and up are never written
            assert dev.vv_gemm_swiglu_dev(P(normed), P(wg), P(wu), None, None, P(gate), T, I_FF, H, st) == 0
        else:
            assert dev.vv_residual_add_dev(P(hidden), P(proj), T * H, st) == 0
            assert dev.vv_rmsnorm_dev(P(hidden), P(n2), P(normed), T, H, EPS, st) == 0
            gemm(normed, wg, gate, I_FF, H)
            gemm(normed, wu, up, I_FF, H)
            assert dev.vv_swiglu_dev(P(gate), P(up), P(gate), T * I_FF, st) == 0
        gemm(gate, wd, proj, H, I_FF)
        if fused:       # the residual add and the next layer's input norm in one launch
            assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n1), P(normed), T, H, EPS, st) == 0
        else:
            assert dev.vv_residual_add_dev(P(hidden), P(proj), T * H, st) == 0
            assert dev.vv_rmsnorm_dev(P(hidden), P(n1), P(normed), T, H, EPS, st) == 0

    def time_layer(fused):
        layer(fused)
        torch.cuda.synchronize()
        per = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            layer(fused)
            e1.record()
            e1.synchronize()
            per.append(e0.elapsed_time(e1))
        per.sort()
        return per[1]

    assert dev.vv_rmsnorm_dev(P(hidden), P(n1), P(normed), T, H, EPS, st) == 0      # layer 0's input norm
    ms_separate = time_layer(False)
    ms = time_layer(True)
    assert bool(torch.isfinite(hidden).all())
    flops = 2.0 * T * H * (2 * QD + 2 * KD + 3 * I_FF) + 4.0 * NQ * HD * T * (T + 1) / 2
    return {"rows": T, "ms_per_layer": ms, "ms_per_layer_reference_api_calls": ms_separate,
            "TFLOPs": flops / ms / 1e9, "layers_assumed": 28, "prompt_tokens_per_s": T / (28 * ms * 1e-3)}


def prefill_chunked_leg(torch, dev, T: int, st: int, chunk: int = 2048) -> dict:
    """One dense decoder layer over a T-row prompt THE WAY THE REFERENCE RUNS IT (decoder.c:1095-1241): chunks of
    at most 2048 rows (7 x 2048 + 113 at T = 14449), each through the layer in decoder_layer_impl's order
    (decoder.c:706-991) - q/k/v projections, bias, RoPE, KV append at the chunk's positions, causal attention of the
    chunk against the cache grown so far, o projection, add + norm, gate/up, SwiGLU, down, add + norm - once on this
    library's fused entry points (q/k/v + bias + RoPE + append in one launch), once on the calls of the reference's
    device.h alone. Random weights; the normed input of every chunk (the previous layer's output) is made before
    the clock starts. Reports ms per layer, per chunk, and the q/k/v leg of a full chunk alone."""
    import ctypes as C
    f16 = dict(dtype=torch.float16, device="cuda")
    QD, KD = NQ * HD, NK * HD
    w = lambda *shape, std: torch.randn(*shape, **f16) * std
    def weights():
        return (w(QD, H, std=H ** -0.5), w(KD, H, std=H ** -0.5), w(KD, H, std=H ** -0.5), w(H, QD, std=QD ** -0.5),
                w(I_FF, H, std=H ** -0.5), w(I_FF, H, std=H ** -0.5), w(H, I_FF, std=I_FF ** -0.5))
    layer0 = weights()
    bq, bk, bv = w(QD, std=0.1), w(KD, std=0.1), w(KD, std=0.1)
    n1, n2 = 1 + w(H, std=0.1), 1 + w(H, std=0.1)
    C_ROWS = min(chunk, T)
    hidden0, normed_in = w(T, H, std=1.0), torch.empty(T, H, **f16)
    hidden = torch.empty(T, H, **f16)
    normed, proj = torch.empty(C_ROWS, H, **f16), torch.empty(C_ROWS, H, **f16)
    q, attn = torch.empty(C_ROWS, QD, **f16), torch.empty(C_ROWS, QD, **f16)
    k, v = torch.empty(C_ROWS, KD, **f16), torch.empty(C_ROWS, KD, **f16)
    gate, up = torch.empty(C_ROWS, I_FF, **f16), torch.empty(C_ROWS, I_FF, **f16)
    kc, vc = torch.empty(T, KD, **f16), torch.empty(T, KD, **f16)
    view = dev.KvView(k=kc.data_ptr(), v=vc.data_ptr(), k_meta=None, v_meta=None, page_table=None, format=0,
                      n_kv_heads=NK, head_dim=HD)
    P = lambda t: t.data_ptr()
    # the context's attention scratch, which the reference's decoder hands to every attention call (decoder.c:755, 893)
    attn_scratch = torch.empty(dev.vv_attn_scratch_bytes(NQ, NK, HD), dtype=torch.uint8, device="cuda")
    rope_table = torch.empty(T, HD // 2, 2, dtype=torch.float32, device="cuda")
    assert dev.vv_rope_table_dev(P(rope_table), T, HD, 0, None, THETA, st) == 0
    assert dev.vv_rmsnorm_dev(P(hidden0), P(n1), P(normed_in), T, H, EPS, st) == 0
    chunks = [(s0, min(chunk, T - s0)) for s0 in range(0, T, chunk)]

    def gemm(x, wt, y, m, n, kk):
        assert dev.vv_gemm_fp16_dev(x, P(wt), P(y), m, n, kk, 1.0, 0.0, st) == 0

    def qkv(start, n, fused, ws=layer0):
        wq, wk, wv = ws[:3]
        x = P(normed_in) + start * H * 2
        if fused:
            # (up to 64 rows the entry point runs the separate launches, which need the k and v buffers)
            kb, vb = (P(k), P(v)) if n <= 64 else (None, None)
            assert dev.vv_gemm_qkv_rope_dev(x, P(wq), P(wk), P(wv), P(bq), P(bk), P(bv), P(q), kb, vb, n, NQ, NK,
                                            HD, H, P(rope_table) + start * HD * 4, P(kc), P(vc), None, start, None,
                                            st) == 0
            return
        gemm(x, wq, q, n, QD, H)
        gemm(x, wk, k, n, KD, H)
        gemm(x, wv, v, n, KD, H)
        assert dev.vv_bias_add_dev(P(q), P(bq), n, QD, st) == 0
        assert dev.vv_bias_add_dev(P(k), P(bk), n, KD, st) == 0
        assert dev.vv_bias_add_dev(P(v), P(bv), n, KD, st) == 0
        assert dev.vv_rope_dev(P(q), n, NQ, HD, start, None, THETA, st) == 0
        assert dev.vv_rope_dev(P(k), n, NK, HD, start, None, THETA, st) == 0
        # the contiguous cache's append (kv_cache.c:238-245): two device copies
        assert dev.vv_dev_memcpy_d2d(P(kc) + start * KD * 2, P(k), n * KD * 2, st) == 0
        assert dev.vv_dev_memcpy_d2d(P(vc) + start * KD * 2, P(v), n * KD * 2, st) == 0

    def one_chunk(start, n, fused, ws=layer0):
        wo, wg, wu, wd = ws[3:]
        h = P(hidden) + start * H * 2
        qkv(start, n, fused, ws)
        assert dev.vv_attn_prefill(2, P(q), C.addressof(view), P(attn), NQ, n, start, start + n, True, P(attn_scratch),
                                   st) == 0
        gemm(P(attn), wo, proj, n, H, QD)
        if fused:
            assert dev.vv_add_rmsnorm_dev(h, P(proj), P(n2), P(normed), n, H, EPS, st) == 0
            assert dev.vv_gemm_swiglu_dev(P(normed), P(wg), P(wu), P(gate), P(up), P(gate), n, I_FF, H, st) == 0
        else:
            assert dev.vv_residual_add_dev(h, P(proj), n * H, st) == 0
            assert dev.vv_rmsnorm_dev(h, P(n2), P(normed), n, H, EPS, st) == 0
            gemm(P(normed), wg, gate, n, I_FF, H)
            gemm(P(normed), wu, up, n, I_FF, H)
            assert dev.vv_swiglu_dev(P(gate), P(up), P(gate), n * I_FF, st) == 0
        gemm(P(gate), wd, proj, n, H, I_FF)
        if fused:       # the residual add and the next layer's input norm in one launch
            assert dev.vv_add_rmsnorm_dev(h, P(proj), P(n1), P(normed), n, H, EPS, st) == 0
        else:
            assert dev.vv_residual_add_dev(h, P(proj), n * H, st) == 0
            assert dev.vv_rmsnorm_dev(h, P(n1), P(normed), n, H, EPS, st) == 0

    def time_layer(fused):
        per, per_chunk = [], None
        for rep in range(4):
            hidden.copy_(hidden0)
            torch.cuda.synchronize()
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(len(chunks) + 1)]
            ev[0].record()
            for i, (s0, n) in enumerate(chunks):
                one_chunk(s0, n, fused)
                ev[i + 1].record()
            ev[-1].synchronize()
            if rep:                                      # the first pass warms up
                per.append((ev[0].elapsed_time(ev[-1]), [ev[i].elapsed_time(ev[i + 1]) for i in range(len(chunks))]))
        per.sort(key=lambda t: t[0])
        return per[len(per) // 2]

    def time_qkv(fused, launches=10):
        s0, n = chunks[-2] if len(chunks) > 1 else chunks[0]
        qkv(s0, n, fused)
        per = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(launches):
                qkv(s0, n, fused)
            e1.record()
            e1.synchronize()
            per.append(e0.elapsed_time(e1) * 1e3 / launches)
        per.sort()
        return n, per[1]

    def time_stream(fused, rows=24, launches=12):
        """A streaming chunk: `rows` rows through the layer on top of the filled cache (the reference's prefill on a
        cache that already holds the session, decoder.c:1112-1114), three layers' weights in rotation (1.4 GB: past
        every cache, as in a 28-layer model)."""
        s0 = T - rows
        for ws in layers:
            one_chunk(s0, rows, fused, ws)
        per = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(launches):
                one_chunk(s0, rows, fused, layers[i % len(layers)])
            e1.record()
            e1.synchronize()
            per.append(e0.elapsed_time(e1) * 1e3 / launches)
        per.sort()
        return per[1]

    ms_api, chunks_api = time_layer(False)
    ms, chunks_ms = time_layer(True)
    assert bool(torch.isfinite(hidden).all())
    rows_qkv, us_qkv = time_qkv(True)
    _, us_qkv_api = time_qkv(False)
    layers = [layer0, weights(), weights()]
    stream_rows = 24
    us_stream, us_stream_api = time_stream(True, stream_rows), time_stream(False, stream_rows)
    del layers
    flops = 2.0 * T * H * (2 * QD + 2 * KD + 3 * I_FF) + 4.0 * NQ * HD * T * (T + 1) / 2
    return {"rows": T, "chunk_rows": [n for _, n in chunks], "ms_per_layer": ms, "ms_per_chunk": chunks_ms,
            "ms_per_layer_reference_api_calls": ms_api, "ms_per_chunk_reference_api_calls": chunks_api,
            "launches_per_chunk": 7, "launches_per_chunk_reference_api_calls": 20,
            "qkv_leg": {"rows": rows_qkv, "us": us_qkv, "us_reference_api_calls": us_qkv_api,
                        "TFLOPs": 2.0 * rows_qkv * (QD + 2 * KD) * H / us_qkv / 1e6},
            "stream_chunk": {"rows": stream_rows, "cache_len": T, "us_per_layer": us_stream,
                             "us_per_layer_reference_api_calls": us_stream_api, "weight_sets_in_rotation": 3},
            "TFLOPs": flops / ms / 1e9, "layers_assumed": 28, "prompt_tokens_per_s": T / (28 * ms * 1e-3)}


def prefill_layer_quant_leg(torch, dev, T: int, st: int, kind: str) -> dict:
    """prefill_layer_leg with quantised projections. kind "w8a8" / "w4a8": int8 activations written by
    the producing op (fused RMSNorm, attention output, fused SwiGLU), biases inside the linears, o and
    down adding into the hidden state through the linear's residual (decoder.c:575-640, 795-932).
    kind "w4a16": INT4 codes against FP16 activations with the decoder's dequant scratch."""
    import ctypes as C
    f16 = dict(dtype=torch.float16, device="cuda")
    QD, KD, G = NQ * HD, NK * HD, 128
    P = lambda t: t.data_ptr() if t is not None else None
    a8, w4 = kind in ("w8a8", "w4a8"), kind in ("w4a16", "w4a8")
    lay = 3 if kind == "w4a8" else 0                        # VV_Q8_W4_MMA for the tiles, else column order
    w = lambda *shape, std: torch.randn(*shape, **f16) * std
    shapes = {"q": (QD, H), "k": (KD, H), "v": (KD, H), "o": (H, QD), "g": (I_FF, H), "u": (I_FF, H), "d": (H, I_FF)}
    wt, sc = {}, {}
    for name, (n, k) in shapes.items():
        if w4:
            wt[name] = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda")
            sc[name] = torch.stack([torch.rand(n, k // G, device="cuda") * 0.004 + 0.002,
                                    torch.randint(0, 16, (n, k // G), device="cuda").float()], dim=-1).half().contiguous()
        else:
            wt[name] = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda")
            sc[name] = torch.rand(n, dtype=torch.float32, device="cuda") * 2e-4 + 1e-4
    bias = {"q": w(QD, std=0.1), "k": w(KD, std=0.1), "v": w(KD, std=0.1)}
    n1, n2 = 1 + w(H, std=0.1), 1 + w(H, std=0.1)
    hidden, normed, proj = w(T, H, std=1.0), torch.empty(T, H, **f16), torch.empty(T, H, **f16)
    q, attn = torch.empty(T, QD, **f16), torch.empty(T, QD, **f16)
    k, v = torch.empty(T, KD, **f16), torch.empty(T, KD, **f16)
    gate, up = torch.empty(T, I_FF, **f16), torch.empty(T, I_FF, **f16)
    xq = torch.empty(T, I_FF, dtype=torch.int8, device="cuda")
    sx = torch.empty(T, dtype=torch.float32, device="cuda")
    xs = torch.empty(T, I_FF // 32, dtype=torch.int32, device="cuda")
    dense = torch.empty(I_FF * H, **f16) if kind == "w4a16" else None
    view = dev.KvView(k=k.data_ptr(), v=v.data_ptr(), k_meta=None, v_meta=None, page_table=None, format=0,
                      n_kv_heads=NK, head_dim=HD)

    def linear(nm, x, y, n, kk, residual=None):
        if kind == "w4a16":
            assert dev.vv_w4a16_gemm_dev(P(x), P(wt[nm]), P(sc[nm]), P(bias.get(nm)), P(y), P(dense), dense.numel() * 2,
                                         T, n, kk, G, st) == 0
        elif kind == "w4a8":
            assert dev.vv_w4a8_linear_dev(P(xq), lay, P(sx), P(xs), P(wt[nm]), P(sc[nm]), G, P(bias.get(nm)),
                                          P(residual), P(y), 0, T, n, kk, 0, st) == 0
        else:
            assert dev.vv_w8a8_linear_dev(P(xq), P(sx), P(wt[nm]), P(sc[nm]), P(bias.get(nm)), P(residual), P(y), 0,
                                          T, n, kk, 0, st) == 0

    def layer():
        if a8:
            assert dev.vv_rmsnorm_q8_dev(P(hidden), P(n1), T, H, EPS, lay, P(xq), P(sx), P(xs), st) == 0
        else:
            assert dev.vv_rmsnorm_dev(P(hidden), P(n1), P(normed), T, H, EPS, st) == 0
        linear("q", normed, q, QD, H)
        linear("k", normed, k, KD, H)
        linear("v", normed, v, KD, H)
        assert dev.vv_rope_qk_dev(P(q), P(k), T, NQ, NK, HD, 0, None, THETA, st) == 0
        assert dev.vv_attn_prefill(2, P(q), C.addressof(view), P(attn), NQ, T, 0, T, True, None, st) == 0
        if a8:
            assert dev.vv_act_quant_dev(P(attn), T, QD, lay, P(xq), P(sx), P(xs), st) == 0
            linear("o", attn, hidden, H, QD, residual=hidden)
            assert dev.vv_rmsnorm_q8_dev(P(hidden), P(n2), T, H, EPS, lay, P(xq), P(sx), P(xs), st) == 0
        else:
            linear("o", attn, proj, H, QD)
            assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n2), P(normed), T, H, EPS, st) == 0
        linear("g", normed, gate, I_FF, H)
        linear("u", normed, up, I_FF, H)
        if a8:
            assert dev.vv_swiglu_q8_dev(P(gate), P(up), T, I_FF, lay, P(xq), P(sx), P(xs), st) == 0
            linear("d", gate, hidden, H, I_FF, residual=hidden)
        else:
            assert dev.vv_swiglu_dev(P(gate), P(up), P(gate), T * I_FF, st) == 0
            linear("d", gate, proj, H, I_FF)
            assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n1), P(normed), T, H, EPS, st) == 0

    layer()
    torch.cuda.synchronize()
    per = []
    for _ in range(3):
        hidden.normal_()                                   # the residual path of the a8 forms grows otherwise
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        layer()
        e1.record()
        e1.synchronize()
        per.append(e0.elapsed_time(e1))
    per.sort()
    ms = per[1]
    assert bool(torch.isfinite(hidden).all())
    ops = 2.0 * T * H * (2 * QD + 2 * KD + 3 * I_FF) + 4.0 * NQ * HD * T * (T + 1) / 2
    return {"weights": kind, "rows": T, "ms_per_layer": ms, "Tops": ops / ms / 1e9, "layers_assumed": 28,
            "prompt_tokens_per_s": T / (28 * ms * 1e-3)}


def decode_token_leg(torch, dev, cache_len: int, layers: int = 28, fused: bool = False) -> dict:
    """One decode step of a dense Qwen2-7B-shaped decoder (random weights, 13 GB of them) on this
    library's entry points alone, in the reference decoder's op order (decoder.c:706-991): per layer
    norm -> q/k/v GEMV -> bias + RoPE at a device-side position -> KV append at that position ->
    split decode attention over `cache_len` positions -> o GEMV -> add+norm -> gate/up GEMV ->
    SwiGLU -> down GEMV -> add+norm. Issued directly, then as one captured graph whose replays
    advance the position on the device. The floor is the weight bytes over the HBM rate."""
    import ctypes as C
    s = C.c_void_p()
    assert dev.vv_dev_stream_create(C.byref(s)) == 0
    st = s.value
    f16 = dict(dtype=torch.float16, device="cuda")
    QD, KD = NQ * HD, NK * HD

    def w(*shape, std):
        return torch.randn(*shape, **f16) * std

    wq, wo = w(layers, QD, H, std=H ** -0.5), w(layers, H, QD, std=QD ** -0.5)
    wk, wv = w(layers, KD, H, std=H ** -0.5), w(layers, KD, H, std=H ** -0.5)
    wg, wu = w(layers, I_FF, H, std=H ** -0.5), w(layers, I_FF, H, std=H ** -0.5)
    wd = w(layers, H, I_FF, std=I_FF ** -0.5)
    bq, bk, bv = w(layers, QD, std=0.1), w(layers, KD, std=0.1), w(layers, KD, std=0.1)
    n_in, n_post = 1 + w(layers + 1, H, std=0.1), 1 + w(layers, H, std=0.1)
    room = cache_len + 256
    kc, vc = w(layers, room, NK, HD, std=1.0), w(layers, room, NK, HD, std=1.0)
    hidden, normed = w(1, H, std=1.0), torch.empty(1, H, **f16)
    q, k, v = torch.empty(1, QD, **f16), torch.empty(1, KD, **f16), torch.empty(1, KD, **f16)
    attn, proj = torch.empty(1, QD, **f16), torch.empty(1, H, **f16)
    gate, up = torch.empty(1, I_FF, **f16), torch.empty(1, I_FF, **f16)
    pos = torch.tensor([cache_len - 1], dtype=torch.int32, device="cuda")    # the new token's position
    nxt = torch.tensor([cache_len], dtype=torch.int32, device="cuda")        # cache length once appended
    scratch = torch.empty(dev.vv_attn_scratch_bytes(NQ, NK, HD), dtype=torch.uint8, device="cuda")
    views = [dev.KvView(k=kc[l].data_ptr(), v=vc[l].data_ptr(), k_meta=None, v_meta=None, page_table=None,
                        format=0, n_kv_heads=NK, head_dim=HD) for l in range(layers)]
    weight_bytes = sum(t.numel() * 2 for t in (wq, wo, wk, wv, wg, wu, wd))
    P = lambda t: t.data_ptr()

    def gemv(x, wt, y, n, kk):
        assert dev.vv_gemm_fp16_dev(P(x), P(wt), P(y), 1, n, kk, 1.0, 0.0, st) == 0

    act = torch.empty(1, I_FF, **f16)
    qkv = []
    for l in range(layers):
        arr = (dev.SkinnyProj * 3)()
        for i, (wt, b, y, n_) in enumerate(((wq, bq, q, QD), (wk, bk, k, KD), (wv, bv, v, KD))):
            arr[i] = dev.SkinnyProj(w=P(wt[l]), scales=None, bias=P(b[l]), y=P(y), N=n_)
        qkv.append(arr)

    def token_fused():
        """The same step on the fused additions: q/k/v with their biases in one launch, gate/up/SwiGLU in one,
        K and V appended by one vv_kv_store_dev."""
        n = 1
        assert dev.vv_rmsnorm_dev(P(hidden), P(n_in[0]), P(normed), 1, H, EPS, st) == 0
        for l in range(layers):
            assert dev.vv_gemv_multi_dev(P(normed), C.addressof(qkv[l]), 3, H, st) == 0
            assert dev.vv_rope_qk_dev(P(q), P(k), 1, NQ, NK, HD, 0, P(pos), THETA, st) == 0
            assert dev.vv_kv_store_dev(P(k), P(v), P(kc[l]), P(vc[l]), None, None, None, False, NK, HD, 0, P(pos), 1,
                                       0, None, st) == 0
            assert dev.vv_attn_decode(2, P(q), C.addressof(views[l]), P(attn), NQ, cache_len, P(nxt),
                                      P(scratch), st) == 0
            gemv(attn, wo[l], proj, H, QD)
            assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n_post[l]), P(normed), 1, H, EPS, st) == 0
            assert dev.vv_gemv_swiglu_dev(P(normed), P(wg[l]), P(wu[l]), P(act), I_FF, H, st) == 0
            gemv(act, wd[l], proj, H, I_FF)
            assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n_in[l + 1]), P(normed), 1, H, EPS, st) == 0
            n += 10
        assert dev.vv_pos_add_dev(P(pos), P(pos), 1, st) == 0
        assert dev.vv_pos_add_dev(P(nxt), P(nxt), 1, st) == 0
        return n + 2

    def token():
        if fused:
            return token_fused()
        n = 1
        assert dev.vv_rmsnorm_dev(P(hidden), P(n_in[0]), P(normed), 1, H, EPS, st) == 0
        for l in range(layers):
            gemv(normed, wq[l], q, QD, H)
            gemv(normed, wk[l], k, KD, H)
            gemv(normed, wv[l], v, KD, H)
            assert dev.vv_bias_rope_qk_dev(P(q), P(k), P(bq[l]), P(bk[l]), 1, NQ, NK, HD, 0, P(pos), THETA, st) == 0
            assert dev.vv_bias_add_dev(P(v), P(bv[l]), 1, KD, st) == 0
            assert dev.vv_dev_memcpy_d2d_at(P(kc[l]), P(k), KD * 2, P(pos), st) == 0
            assert dev.vv_dev_memcpy_d2d_at(P(vc[l]), P(v), KD * 2, P(pos), st) == 0
            assert dev.vv_attn_decode(2, P(q), C.addressof(views[l]), P(attn), NQ, cache_len, P(nxt),
                                      P(scratch), st) == 0
            gemv(attn, wo[l], proj, H, QD)
            assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n_post[l]), P(normed), 1, H, EPS, st) == 0
            gemv(normed, wg[l], gate, I_FF, H)
            gemv(normed, wu[l], up, I_FF, H)
            assert dev.vv_swiglu_dev(P(gate), P(up), P(gate), I_FF, st) == 0
            gemv(gate, wd[l], proj, H, I_FF)
            assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n_in[l + 1]), P(normed), 1, H, EPS, st) == 0
            n += 16
        assert dev.vv_pos_add_dev(P(pos), P(pos), 1, st) == 0
        assert dev.vv_pos_add_dev(P(nxt), P(nxt), 1, st) == 0
        return n + 2

    torch.cuda.synchronize()
    launches = token()
    assert dev.vv_dev_stream_sync(st) == 0
    reps = 10
    t0 = time.perf_counter()
    for _ in range(reps):
        token()
    assert dev.vv_dev_stream_sync(st) == 0
    eager = (time.perf_counter() - t0) / reps
    assert dev.vv_dev_graph_begin(st) == 0
    token()
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(st, C.byref(g)) == 0 and g.value
    for _ in range(2):
        assert dev.vv_dev_graph_launch(g.value, st) == 0
    assert dev.vv_dev_stream_sync(st) == 0
    before = int(pos.item())
    t0 = time.perf_counter()
    for _ in range(reps):
        assert dev.vv_dev_graph_launch(g.value, st) == 0
    assert dev.vv_dev_stream_sync(st) == 0
    replay = (time.perf_counter() - t0) / reps
    assert int(pos.item()) == before + reps and int(nxt.item()) == before + reps + 1
    assert bool(torch.isfinite(normed).all())
    dev.vv_dev_graph_destroy(g.value)
    dev.vv_dev_stream_destroy(st)
    return {"layers": layers, "cache_len": cache_len, "launches": launches, "weight_bytes": weight_bytes,
            "entry_points": "fused additions" if fused else "reference API",
            "eager_ms": eager * 1e3, "graph_ms": replay * 1e3, "tokens_per_s": 1.0 / replay,
            "weight_GBps": weight_bytes / replay / 1e9,
            "frac_of_hbm_peak": weight_bytes / replay / 1e9 / HBM_PEAK_GBPS}


def decode_token_quant_leg(torch, dev, cache_len: int, kind: str, layers: int = 28) -> dict:
    """The decode step of decode_token_leg with quantised projections, in the reference decoder's op
    order for them. kind "w4a16": INT4 codes against FP16 activations (decoder.c:412-422, 512-520:
    fused q/k/v and gate/up GEMVs with their biases). kind "w8a8" / "w4a8": int8 activations written
    by the producing op (RMSNorm, attention output, SwiGLU), o and down adding into the hidden state
    through the linear's residual (decoder.c:575-640, 795-932). Random weights and codes."""
    import ctypes as C
    s = C.c_void_p()
    assert dev.vv_dev_stream_create(C.byref(s)) == 0
    st = s.value
    f16 = dict(dtype=torch.float16, device="cuda")
    QD, KD, G = NQ * HD, NK * HD, 128
    P = lambda t: t.data_ptr() if t is not None else None
    a8, w4 = kind in ("w8a8", "w4a8"), kind in ("w4a16", "w4a8")
    lay = 2 if kind == "w4a8" else 0                        # VV_Q8_W4_GEMV for one row, else column order

    def w(*shape, std):
        return torch.randn(*shape, **f16) * std

    shapes = {"q": (QD, H), "k": (KD, H), "v": (KD, H), "o": (H, QD), "g": (I_FF, H), "u": (I_FF, H), "d": (H, I_FF)}
    wt, sc, weight_bytes = {}, {}, 0
    for name, (n, k) in shapes.items():
        if w4:
            wt[name] = torch.randint(0, 256, (layers, n, k // 2), dtype=torch.uint8, device="cuda")
            sc[name] = torch.stack([torch.rand(layers, n, k // G, device="cuda") * 0.004 + 0.002,
                                    torch.randint(0, 16, (layers, n, k // G), device="cuda").float()],
                                   dim=-1).half().contiguous()
        else:
            wt[name] = torch.randint(-127, 128, (layers, n, k), dtype=torch.int8, device="cuda")
            sc[name] = torch.rand(layers, n, dtype=torch.float32, device="cuda") * 2e-4 + 1e-4
        weight_bytes += wt[name].numel() * wt[name].element_size() + sc[name].numel() * sc[name].element_size()
    bq, bk, bv = w(layers, QD, std=0.1), w(layers, KD, std=0.1), w(layers, KD, std=0.1)
    n_in, n_post = 1 + w(layers + 1, H, std=0.1), 1 + w(layers, H, std=0.1)
    room = cache_len + 256
    kc, vc = w(layers, room, NK, HD, std=1.0), w(layers, room, NK, HD, std=1.0)
    hidden, normed = w(1, H, std=1.0), torch.empty(1, H, **f16)
    q, k, v = torch.empty(1, QD, **f16), torch.empty(1, KD, **f16), torch.empty(1, KD, **f16)
    attn, proj = torch.empty(1, QD, **f16), torch.empty(1, H, **f16)
    gate, up, act = torch.empty(1, I_FF, **f16), torch.empty(1, I_FF, **f16), torch.empty(1, I_FF, **f16)
    xq = torch.empty(1, I_FF, dtype=torch.int8, device="cuda")
    sx = torch.empty(1, dtype=torch.float32, device="cuda")
    xs = torch.empty(1, I_FF // 32, dtype=torch.int32, device="cuda")
    pos = torch.tensor([cache_len - 1], dtype=torch.int32, device="cuda")
    nxt = torch.tensor([cache_len], dtype=torch.int32, device="cuda")
    scratch = torch.empty(dev.vv_attn_scratch_bytes(NQ, NK, HD), dtype=torch.uint8, device="cuda")
    views = [dev.KvView(k=kc[l].data_ptr(), v=vc[l].data_ptr(), k_meta=None, v_meta=None, page_table=None,
                        format=0, n_kv_heads=NK, head_dim=HD) for l in range(layers)]

    qkv, gu = [], []
    for l in range(layers):
        if a8:
            a3, a2 = (dev.I8Proj * 3)(), (dev.I8Proj * 2)()
            for i, (nm, b, y, n_) in enumerate((("q", bq, q, QD), ("k", bk, k, KD), ("v", bv, v, KD))):
                a3[i] = dev.I8Proj(P(wt[nm][l]), P(sc[nm][l]), P(sc[nm][l]), P(b[l]), P(y), n_)
            for i, (nm, y) in enumerate((("g", gate), ("u", up))):
                a2[i] = dev.I8Proj(P(wt[nm][l]), P(sc[nm][l]), P(sc[nm][l]), None, P(y), I_FF)
        else:
            a3, a2 = (dev.W4A16Proj * 3)(), (dev.W4A16Proj * 2)()
            for i, (nm, b, y, n_) in enumerate((("q", bq, q, QD), ("k", bk, k, KD), ("v", bv, v, KD))):
                a3[i] = dev.W4A16Proj(P(wt[nm][l]), P(sc[nm][l]), P(b[l]), P(y), n_)
            for i, (nm, y) in enumerate((("g", gate), ("u", up))):
                a2[i] = dev.W4A16Proj(P(wt[nm][l]), P(sc[nm][l]), None, P(y), I_FF)
        qkv.append(a3)
        gu.append(a2)

    def a8_linear(nm, l, n, kk, residual, y):
        if w4:
            assert dev.vv_w4a8_linear_dev(P(xq), lay, P(sx), P(xs), P(wt[nm][l]), P(sc[nm][l]), G, None, P(residual),
                                          P(y), 0, 1, n, kk, 0, st) == 0
        else:
            assert dev.vv_w8a8_linear_dev(P(xq), P(sx), P(wt[nm][l]), P(sc[nm][l]), None, P(residual), P(y), 0, 1, n,
                                          kk, 0, st) == 0

    def common_attention(l):
        assert dev.vv_rope_qk_dev(P(q), P(k), 1, NQ, NK, HD, 0, P(pos), THETA, st) == 0
        assert dev.vv_kv_store_dev(P(k), P(v), P(kc[l]), P(vc[l]), None, None, None, False, NK, HD, 0, P(pos), 1, 0,
                                   None, st) == 0
        assert dev.vv_attn_decode(2, P(q), C.addressof(views[l]), P(attn), NQ, cache_len, P(nxt), P(scratch), st) == 0
        return 3

    def token():
        n = 1
        if a8:
            assert dev.vv_rmsnorm_q8_dev(P(hidden), P(n_in[0]), 1, H, EPS, lay, P(xq), P(sx), P(xs), st) == 0
            for l in range(layers):
                assert dev.vv_i8_linear_multi_dev(P(xq), lay, P(sx), P(xs), 1 if w4 else 0, C.addressof(qkv[l]), 3, G,
                                                  1, H, st) == 0
                n += 1 + common_attention(l)
                assert dev.vv_act_quant_dev(P(attn), 1, QD, lay, P(xq), P(sx), P(xs), st) == 0
                a8_linear("o", l, H, QD, hidden, hidden)
                assert dev.vv_rmsnorm_q8_dev(P(hidden), P(n_post[l]), 1, H, EPS, lay, P(xq), P(sx), P(xs), st) == 0
                assert dev.vv_i8_linear_multi_dev(P(xq), lay, P(sx), P(xs), 1 if w4 else 0, C.addressof(gu[l]), 2, G,
                                                  1, H, st) == 0
                assert dev.vv_swiglu_q8_dev(P(gate), P(up), 1, I_FF, lay, P(xq), P(sx), P(xs), st) == 0
                a8_linear("d", l, H, I_FF, hidden, hidden)
                assert dev.vv_rmsnorm_q8_dev(P(hidden), P(n_in[l + 1]), 1, H, EPS, lay, P(xq), P(sx), P(xs), st) == 0
                n += 7
        else:
            assert dev.vv_rmsnorm_dev(P(hidden), P(n_in[0]), P(normed), 1, H, EPS, st) == 0
            for l in range(layers):
                assert dev.vv_w4a16_gemv_multi_dev(P(normed), C.addressof(qkv[l]), 3, H, G, st) == 0
                n += 1 + common_attention(l)
                assert dev.vv_w4a16_gemv_dev(P(attn), P(wt["o"][l]), P(sc["o"][l]), None, P(proj), H, QD, G, st) == 0
                assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n_post[l]), P(normed), 1, H, EPS, st) == 0
                assert dev.vv_w4a16_gemv_multi_dev(P(normed), C.addressof(gu[l]), 2, H, G, st) == 0
                assert dev.vv_swiglu_dev(P(gate), P(up), P(act), I_FF, st) == 0
                assert dev.vv_w4a16_gemv_dev(P(act), P(wt["d"][l]), P(sc["d"][l]), None, P(proj), H, I_FF, G, st) == 0
                assert dev.vv_add_rmsnorm_dev(P(hidden), P(proj), P(n_in[l + 1]), P(normed), 1, H, EPS, st) == 0
                n += 6
        assert dev.vv_pos_add_dev(P(pos), P(pos), 1, st) == 0
        assert dev.vv_pos_add_dev(P(nxt), P(nxt), 1, st) == 0
        return n + 2

    torch.cuda.synchronize()
    calls = token()
    assert dev.vv_dev_stream_sync(st) == 0
    reps = 10
    t0 = time.perf_counter()
    for _ in range(reps):
        token()
    assert dev.vv_dev_stream_sync(st) == 0
    eager = (time.perf_counter() - t0) / reps
    assert dev.vv_dev_graph_begin(st) == 0
    token()
    g = C.c_void_p()
    assert dev.vv_dev_graph_end(st, C.byref(g)) == 0 and g.value
    for _ in range(2):
        assert dev.vv_dev_graph_launch(g.value, st) == 0
    assert dev.vv_dev_stream_sync(st) == 0
    before = int(pos.item())
    t0 = time.perf_counter()
    for _ in range(reps):
        assert dev.vv_dev_graph_launch(g.value, st) == 0
    assert dev.vv_dev_stream_sync(st) == 0
    replay = (time.perf_counter() - t0) / reps
    assert int(pos.item()) == before + reps
    assert bool(torch.isfinite(hidden).all())
    dev.vv_dev_graph_destroy(g.value)
    dev.vv_dev_stream_destroy(st)
    return {"weights": kind, "layers": layers, "cache_len": cache_len, "calls": calls, "weight_bytes": weight_bytes,
            "eager_ms": eager * 1e3, "graph_ms": replay * 1e3, "tokens_per_s": 1.0 / replay,
            "weight_GBps": weight_bytes / replay / 1e9,
            "frac_of_hbm_peak": weight_bytes / replay / 1e9 / HBM_PEAK_GBPS}


def cpu_baseline(rows: int) -> dict:
    """The CPU path of the same step on `rows` rows: warm-up, then best of five
    (bench/benchmark.c:197-211). FP32 activations, so its byte count is its own."""
    import ctypes as C

    import numpy as np

    import oracle

    f32p, i32p = C.POINTER(C.c_float), C.POINTER(C.c_int32)
    use_ref = oracle.ref is not None
    if use_ref:
        threads = oracle.ref.vv_cpu_threads()     # one per physical core, pinned; OMP_NUM_THREADS wins
        simd = oracle.ref.vv_cpu_simd_name().decode()
    else:
        threads, simd = oracle.lib.vvo_threads(), "scalar"
    vocab = V                                      # the whole [152064, 3584] table: 1.09 GB of host memory
    table = oracle.normal_f16((vocab, H), 1, std=0.02)
    ids = oracle.ids(rows, 2, vocab)
    w = oracle.normal_f16((H,), 3, mean=1.0, std=0.1)
    hidden = np.empty((rows, H), np.float32)
    normed = np.empty((rows, H), np.float32)
    resid = oracle.normal_f32((rows, H), 4)
    x = oracle.normal_f32((rows, H), 5)
    q = oracle.normal_f32((rows, NQ, HD), 6)
    k = oracle.normal_f32((rows, NK, HD), 7)
    gate = oracle.normal_f32((rows, I_FF), 8, std=2.0)
    up = oracle.normal_f32((rows, I_FF), 9, std=2.0)
    out = np.empty((rows, I_FF), np.float32)

    def p(a, ty=f32p):
        return a.ctypes.data_as(ty)

    if use_ref:
        r = oracle.ref
        steps = {
            "gather+norm": lambda: (r.vv_embedding_cpu(table.ctypes.data, p(ids, i32p), p(hidden), rows, H),
                                    r.vv_rmsnorm_cpu(p(hidden), w.ctypes.data, p(normed), rows, H, C.c_float(EPS))),
            "add+norm": lambda: (r.vv_residual_add_cpu(p(resid), p(x), rows * H),
                                 r.vv_rmsnorm_cpu(p(resid), w.ctypes.data, p(normed), rows, H, C.c_float(EPS))),
            "rope": lambda: (r.vv_rope_cpu(p(q), rows, NQ, HD, 0, C.c_float(THETA)),
                             r.vv_rope_cpu(p(k), rows, NK, HD, 0, C.c_float(THETA))),
            "swiglu": lambda: (r.vv_swiglu_cpu(p(gate), p(up), p(out), rows * I_FF),),
        }
    else:
        u16p = C.POINTER(C.c_uint16)
        o = oracle.lib
        steps = {
            "gather+norm": lambda: (o.vvo_embedding_f32(p(table, u16p), p(ids, i32p), p(hidden), rows, H),
                                    o.vvo_rmsnorm_f32(p(hidden), p(w, u16p), p(normed), rows, H, EPS)),
            "add+norm": lambda: (o.vvo_residual_add_f32(p(resid), p(x), rows * H),
                                 o.vvo_rmsnorm_f32(p(resid), p(w, u16p), p(normed), rows, H, EPS)),
            "rope": lambda: (o.vvo_rope_f32(p(q), rows, NQ, HD, 0, THETA),
                             o.vvo_rope_f32(p(k), rows, NK, HD, 0, THETA)),
            "swiglu": lambda: (o.vvo_swiglu_f32(p(gate), p(up), p(out), rows * I_FF),),
        }
    # the CPU path's own traffic: FP32 activations, FP16 weights/table
    cpu_bytes = {
        "gather+norm": rows * (4 + 2 * H) + 4 * rows * H + 8 * rows * H + 2 * H,
        "add+norm": 12 * rows * H + 8 * rows * H + 2 * H,
        "rope": 8 * rows * (NQ + NK) * HD,
        "swiglu": 12 * rows * I_FF,
    }
    per, total = {}, 0.0
    for name in KERNELS:
        fn = steps[name]
        assert all(rc == 0 for rc in fn())                  # warm-up
        best = float("inf")
        for _ in range(5):
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
        per[name] = {"ms": best * 1e3, "rows_per_s": rows / best,
                     "GBps_own_bytes": cpu_bytes[name] / best / 1e9}
        total += best
        log(f"  cpu {name:12s} {best * 1e3:9.2f} ms  {rows / best:12.0f} rows/s")
    return {
        "value": sum(cpu_bytes.values()) / total / 1e9,
        "unit": "GB/s (on the CPU path's own FP32 byte count)",
        "cores": threads,
        "kind": "reference" if use_ref else "port",
        "simd": simd,
        "sample": f"the same step on {rows} of {T_FULL} rows (the whole {vocab}-row embedding table), "
                  "best of 5 after a warm-up call",
        "rows_per_s": rows / total,
        "ms_per_step_sample": total * 1e3,
        "kernels": per,
    }


def layer_legs(torch, dev, T: int, st: int, args, fp16_only: bool) -> dict:
    """The GEMM / attention / whole-layer legs reported under 'layer' (none of them part of `value`)."""
    layer = layer_leg(torch, dev, T, st, fp16_only)
    for name, d in list(layer["gemm"].items()) + list(layer.get("gemm_chunk", {}).items()):
        log(f"  gemm {name:13s} M={d['M']} N={d['N']} K={d['K']}: {d['us']:9.1f} us {d['TFLOPs']:7.1f} TFLOP/s "
            f"({100 * d['frac_of_mfma_peak']:.1f} % of the FP16 matrix peak)")
    for name, d in layer.get("gemm_swiglu", {}).items():
        log(f"  gemm gate+up+swiglu M={d['M']} N={d['N']} K={d['K']}: {d['us']:9.1f} us {d['TFLOPs']:7.1f} TFLOP/s "
            f"({100 * d['frac_of_mfma_peak']:.1f} % of the FP16 matrix peak); as two GEMMs and SwiGLU "
            f"{d['us_two_gemms_and_swiglu']:.1f} us")
    for name, d in layer["gemv"].items():
        log(f"  gemv {name:13s} N={d['N']} K={d['K']}: {d['us']:7.2f} us {d['GBps']:7.1f} GB/s")
    for kind in () if fp16_only else ("w8a8", "w4a8"):
        for name, d in layer[kind].items():
            log(f"  {kind} {name:13s} M={d['M']} N={d['N']} K={d['K']}: {d['us']:9.1f} us {d['TOPs']:7.1f} TOP/s "
                f"({100 * d['frac_of_mfma_peak']:.1f} % of the int8 matrix peak)")
        for name, d in layer[kind + "_gemv"].items():
            log(f"  {kind} gemv {name:13s} N={d['N']} K={d['K']}: {d['us']:7.2f} us {d['GBps']:7.1f} GB/s")
    for name, d in layer.get("w4a8_chunk", {}).items():
        log(f"  w4a8 {d['M']} rows {name:13s} N={d['N']} K={d['K']}: {d['us']:7.2f} us {d['GBps']:7.1f} GB/s")
    for name, d in layer.get("w4a16", {}).items():
        log(f"  w4a16 {name:13s} M={d['M']} N={d['N']} K={d['K']}: {d['us']:9.1f} us {d['TFLOPs']:7.1f} TFLOP/s "
            f"({100 * d['frac_of_mfma_peak']:.1f} % of the FP16 matrix peak)")
    for name, d in layer.get("w4a16_gemv", {}).items():
        log(f"  w4a16 gemv {name:13s} N={d['N']} K={d['K']}: {d['us']:7.2f} us {d['GBps']:7.1f} GB/s")
    for name, d in layer.get("w4a16_chunk", {}).items():
        log(f"  w4a16 {d['M']} rows {name:13s} N={d['N']} K={d['K']}: {d['us']:7.2f} us {d['GBps']:7.1f} GB/s")
    for name, d in layer.get("weight_only", {}).items():
        log(f"  weight-only {name:18s} N={d['N']} K={d['K']}: one row {d['M1_us']:7.2f} us {d['M1_GBps']:7.1f} GB/s, "
            f"29 rows {d['M29_us']:7.2f} us, dequantise {d['dequant_us']:7.2f} us {d['dequant_GBps']:7.1f} GB/s")
    d = layer["attn_prefill"]
    log(f"  attention prefill T={T}: {d['us']:9.1f} us {d['TFLOPs']:7.1f} TFLOP/s "
        f"({100 * d['frac_of_mfma_peak']:.1f} % of the FP16 matrix peak)")
    if "attn_prefill_chunk" in layer:
        d = layer["attn_prefill_chunk"]
        log(f"  attention prefill, rows {d['q_offset']}..{T - 1} against {T} keys: {d['us']:9.1f} us "
            f"{d['TFLOPs']:7.1f} TFLOP/s ({100 * d['frac_of_mfma_peak']:.1f} % of the FP16 matrix peak)")
    d = layer["attn_decode"]
    log(f"  attention decode, cache {T}: {d['us']:7.2f} us {d['GBps']:7.1f} GB/s "
        f"(replayed from a graph: {d['graph_us']:.2f} us {d['graph_GBps']:.1f} GB/s)")
    if not fp16_only:
        d = layer["attn_prefill_fp8"]
        log(f"  attention prefill, FP8 cache: {d['us']:9.1f} us {d['TFLOPs']:7.1f} TFLOP/s")
        d = layer["attn_decode_fp8"]
        log(f"  attention decode, FP8 cache {T}: {d['us']:7.2f} us {d['GBps']:7.1f} GB/s")
        d = layer["bitnet"]
        log("  BitNet (1536 / 8960 / 151936): " + ", ".join(f"{k} {v:.1f}" for k, v in d.items()))
        d = layer["vae"]
        log("  Conv-VAE ops (512 channels x 24000 columns): " + ", ".join(f"{k} {v:.1f}" for k, v in d.items()))
    layer["prefill_layer"] = d = prefill_layer_leg(torch, dev, T, st)
    log(f"  prefill layer, T={T}: {d['ms_per_layer']:.2f} ms ({d['TFLOPs']:.0f} TFLOP/s over GEMMs + attention; "
        f"{d['ms_per_layer_reference_api_calls']:.2f} ms on the calls of the reference's device.h alone); "
        f"28 layers = {d['prompt_tokens_per_s']:.0f} prompt tokens/s")
    torch.cuda.empty_cache()
    layer["prefill_chunked"] = d = prefill_chunked_leg(torch, dev, T, st)
    log(f"  prefill layer in {len(d['chunk_rows'])} chunks of <= 2048 rows (the reference's launch pattern), T={T}: "
        f"{d['ms_per_layer']:.2f} ms ({d['TFLOPs']:.0f} TFLOP/s; {d['ms_per_layer_reference_api_calls']:.2f} ms on the "
        f"calls of the reference's device.h alone); q/k/v + bias + RoPE + append of {d['qkv_leg']['rows']} rows "
        f"{d['qkv_leg']['us']:.1f} us in one launch, {d['qkv_leg']['us_reference_api_calls']:.1f} us in ten; "
        f"28 layers = {d['prompt_tokens_per_s']:.0f} prompt tokens/s")
    sc = d["stream_chunk"]
    log(f"  a streaming chunk of {sc['rows']} rows on top of the {sc['cache_len']}-position cache, one layer (three layers' "
        f"weights in rotation): {sc['us_per_layer']:.1f} us ({sc['us_per_layer_reference_api_calls']:.1f} us on the calls "
        f"of the reference's device.h alone)")
    for kind in () if fp16_only else ("w8a8", "w4a8", "w4a16"):
        torch.cuda.empty_cache()
        layer["prefill_layer_" + kind] = d = prefill_layer_quant_leg(torch, dev, T, st, kind)
        log(f"  prefill layer, {kind} projections: {d['ms_per_layer']:.2f} ms ({d['Tops']:.0f} TOP/s over linears + "
            f"attention); 28 layers = {d['prompt_tokens_per_s']:.0f} prompt tokens/s")
    if not args.no_token:
        layer["decode_token"] = d = decode_token_leg(torch, dev, T)
        log(f"  decode token, {d['layers']} layers, cache {T}: {d['launches']} launches, eager {d['eager_ms']:.3f} ms, "
            f"graph {d['graph_ms']:.3f} ms = {d['tokens_per_s']:.0f} tokens/s, weights at {d['weight_GBps']:.0f} GB/s "
            f"({100 * d['frac_of_hbm_peak']:.1f} % of peak)")
        layer["decode_token_fused"] = d = decode_token_leg(torch, dev, T, fused=True)
        log(f"  decode token, fused additions: {d['launches']} launches, eager {d['eager_ms']:.3f} ms, "
            f"graph {d['graph_ms']:.3f} ms = {d['tokens_per_s']:.0f} tokens/s, weights at {d['weight_GBps']:.0f} GB/s "
            f"({100 * d['frac_of_hbm_peak']:.1f} % of peak)")

    for kind in () if fp16_only or args.no_token else ("w4a16", "w8a8", "w4a8"):
        torch.cuda.empty_cache()
        layer["decode_token_" + kind] = d = decode_token_quant_leg(torch, dev, T, kind)
        log(f"  decode token, {kind} projections: {d['calls']} calls, eager {d['eager_ms']:.3f} ms, "
            f"graph {d['graph_ms']:.3f} ms = {d['tokens_per_s']:.0f} tokens/s, weights at "
            f"{d['weight_GBps']:.0f} GB/s ({100 * d['frac_of_hbm_peak']:.1f} % of peak)")
    return layer


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--rows", type=int, default=T_FULL, help="prompt length T")
    ap.add_argument("--sets", type=int, default=3, help="rotating buffer sets")
    ap.add_argument("--launches", type=int, default=20, help="back-to-back launches per event pair")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-config (smaller T) leg")
    ap.add_argument("--only", default=None, help="time only this kernel (profiling aid)")
    ap.add_argument("--reps", type=int, default=5, help="event-timed repetitions per kernel")
    ap.add_argument("--unfused", action="store_true",
                    help="also time the unfused reference-API calls and the int8-activation fused "
                         "forms (reported under 'unfused'; not part of the step)")
    ap.add_argument("--layer", action="store_true",
                    help="also time the dense GEMM and attention entry points at the layer's shapes "
                         "(reported under 'layer'; not part of the step)")
    ap.add_argument("--layer-fp16", action="store_true",
                    help="like --layer, but only the FP16 GEMM and attention legs and the whole-layer / whole-token "
                         "figures built on them (no quantised, BitNet or Conv-VAE legs): short enough to profile")
    ap.add_argument("--no-token", action="store_true",
                    help="with --layer / --layer-fp16: skip the whole-token decode legs (thousands of small launches)")
    ap.add_argument("--no-layer", action="store_true",
                    help="skip the FP16 GEMM and attention legs that a plain run reports under 'layer' "
                         "(the --layer-fp16 legs without the whole-token ones)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain 256 MiB copy kernel (vv_dev_memcpy_d2d_at at index 0) "
                         "five times: the known-size reference for rocprofv3 byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every op is row-independent and this build uses no "
              "second device; run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    from __graft_entry__ import load_device

    dev = load_device()                              # raises if the HIP library is not built
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU: there is no CPU fallback for the HIP backend")
    torch.cuda.set_device(0)
    T = args.rows
    name_buf = torch.cuda.get_device_name(0)
    log(f"device: {name_buf}; T={T}, sets={args.sets}")
    wl = Workload(torch, dev, T, args.sets)
    st = torch.cuda.current_stream().cuda_stream
    if args.calibrate:
        n = 256 << 20
        src = torch.ones(n, dtype=torch.uint8, device="cuda")
        dst = torch.zeros(n, dtype=torch.uint8, device="cuda")
        idx = torch.zeros(1, dtype=torch.int32, device="cuda")
        for _ in range(5):
            assert dev.vv_dev_memcpy_d2d_at(dst.data_ptr(), src.data_ptr(), n, idx.data_ptr(), st) == 0
        torch.cuda.synchronize()
        assert bool((dst == 1).all())
        del src, dst
    bytes_per = algorithmic_bytes(T)
    kernels = [args.only] if args.only else KERNELS

    # ── whole step: W warm-up steps, then exactly K timed steps ──
    for i in range(args.warmup):
        for name in kernels:
            wl.launch(name, i, st)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        for name in kernels:
            wl.launch(name, i, st)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    step_bytes = sum(bytes_per[n] for n in kernels)
    value = step_bytes / (wall / args.steps) / 1e9
    log(f"step: {ms_per_step:.4f} ms, {value:.1f} GB/s over {step_bytes / 1e6:.1f} MB")

    # ── per kernel, HIP events on the launch stream ──
    per = {}
    for name in kernels:
        best, med = time_kernel(torch, wl, name, args.launches, args.reps, st)
        per[name] = {
            "bytes": bytes_per[name],
            "us_median": med * 1e6, "us_best": best * 1e6,
            "GBps": bytes_per[name] / med / 1e9,
            "frac_of_peak": bytes_per[name] / med / 1e9 / HBM_PEAK_GBPS,
            "rows_per_s": T / med,
        }
        log(f"  {name:12s} {med * 1e6:9.2f} us  {per[name]['GBps']:8.1f} GB/s  "
            f"{100 * per[name]['frac_of_peak']:5.1f} % of peak  {T / med:12.0f} rows/s")

    unfused = {}
    if args.unfused:
        for name in UNFUSED:
            best, med = time_kernel(torch, wl, name, args.launches, args.reps, st)
            unfused[name] = {"bytes": bytes_per[name], "us_median": med * 1e6,
                             "GBps": bytes_per[name] / med / 1e9,
                             "frac_of_peak": bytes_per[name] / med / 1e9 / HBM_PEAK_GBPS}
            log(f"  {name:12s} {med * 1e6:9.2f} us  {unfused[name]['GBps']:8.1f} GB/s  "
                f"{100 * unfused[name]['frac_of_peak']:5.1f} % of peak  (not part of the step)")

    layer = {}
    # a plain run carries the FP16 GEMM / attention figures too (a dozen seconds; never part of `value`)
    default_layer = not (args.layer or args.layer_fp16 or args.no_layer or args.only)
    if default_layer:
        args.no_token = True
    if args.layer or args.layer_fp16:
        layer = layer_legs(torch, dev, T, st, args, not args.layer)
    elif default_layer:
        try:                                  # the line's own figures must not depend on these legs
            layer = layer_legs(torch, dev, T, st, args, True)
        except Exception as e:  # noqa: BLE001
            log(f"  layer legs failed: {e!r}")
            layer = {"error": repr(e)}

    # ── BASELINE.json's config shapes and the 2048-row prefill chunk, cold ──
    configs = []
    if not args.only and not args.no_configs:
        configs = configs_leg(torch, dev, wl, st)

    # ── decode shape (T = 1): launch-bound, reported as microseconds per launch ──
    decode = {}
    if not args.only:
        wl1 = Workload(torch, dev, 1, 1, table=wl.table, weight=wl.weight)
        for name in KERNELS:
            best, med = time_kernel(torch, wl1, name, 200, 3, st)
            decode[name] = {"us_median": med * 1e6, "bytes": algorithmic_bytes(1)[name]}
        log("  decode (T=1) us per launch: " +
            ", ".join(f"{n} {d['us_median']:.2f}" for n, d in decode.items()))

    # ── the decode step's layer ops as one captured graph (28 layers x 5 launches) ──
    graph = {}
    if not args.only:
        graph = decode_graph_leg(torch, dev, wl1)
        log(f"  decode graph: {graph['launches']} launches, eager {graph['eager_us']:.1f} us, "
            f"graph replay {graph['replay_us']:.1f} us ({graph['replay_us_per_launch']:.2f} us/launch)")

    dominant = max(kernels, key=lambda n: bytes_per[n])
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get(dominant, {}).get("hbm_bytes_per_launch")
    result = {
        "metric": "achieved HBM GB/s (% of MI355X peak) for RMSNorm/RoPE/SwiGLU at T=14449",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "storage_dtype": "f16", "data": "synthetic",
        "config": {"workload": f"Qwen2-7B fused layer kernels, one prefill pass at T={T}: "
                               "embedding gather+RMSNorm, residual-add+RMSNorm, RoPE(Q,K), SwiGLU",
                   "hidden": H, "intermediate": I_FF, "vocab": V, "q_heads": NQ, "kv_heads": NK,
                   "head_dim": HD, "rows": T, "buffer_sets": args.sets},
        "pct_of_peak": 100.0 * value / HBM_PEAK_GBPS,
        "rows_per_s": T / (wall / args.steps),
        "kernels": per,
        "roofline": {"kernel": dominant, "bound": "hbm", "achieved": per[dominant]["GBps"],
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": per[dominant]["frac_of_peak"], "traffic": traffic,
                     "traffic_source": "profiles/pmc_traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                       "of this kernel at this shape, recorded earlier, not measured in this run"},
    }
    if configs:
        result["configs"] = configs
    if unfused:
        result["unfused"] = unfused
    if layer:
        result["layer"] = layer
    if decode:
        result["decode_T1_us"] = decode
    if graph:
        result["decode_graph"] = graph
    if not args.no_cpu:
        log(f"cpu baseline on {CPU_SAMPLE_ROWS} rows ...")
        result["cpu_baseline"] = cpu_baseline(CPU_SAMPLE_ROWS)
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
