#!/usr/bin/env python3
"""Benchmark of the HLQ LUT GEMV hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-decode]

Workload: the LLaMA-3-8B layer-shape sweep at HLQ w2g128, batch 1.
One "step" streams the seven projections (q, k, v, o, gate, up, down) of all 32 layers --
224 GEMVs over 224 distinct random weight sets, 2.07 GB of packed planes + scales + zeros,
far more than the 256 MB Infinity Cache, so every step reads its weights from HBM.  Inputs
are resident in HBM before the timed region.  The step is captured once in a HIP graph and
replayed, so the figure is GPU throughput, not Python launch rate.  Defaults: K = 4000 timed steps after
W = 10 (about four seconds of continuous GPU work per leg; the whole run takes about a minute).

Prints ONE JSON line.  `value` is algorithmic bytes per step / time per step in GB/s
(bytes = planes + fp16 scales + fp16 zeros + x + y per GEMV).  `per_shape` holds the
per-shape latency / bandwidth of the four distinct (K, N), each measured over a ring of
weight sets larger than 512 MB.  `roofline` is for the dominant kernel (the 4096x14336
gate/up GEMV); `cpu_baseline` times the C port of the reference's CPU LUT kernel
(oracle/lut_gemv_ref.c, AVX2 build) on this machine's host cores over a bounded sample.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "hlq_gemv_w2g128_4096x14336_hbm_traffic.md")
TRACE_PROFILE = os.path.join(ROOT, "profiles", "hlq_gemv_w2g128_sweep_kernel_trace.md")
KERNEL_SOURCES = ["hlq_gemv.hip", "hlq_gemv_dev.h", "hlq_gemv_index.h", "hlq_layout.h"]     # what the dominant kernel is compiled from


def kernel_source_hash():
    """First 16 hex digits of the SHA-256 of the dominant kernel's sources: the committed counter summaries carry the
    hash of the sources they were measured on, so a figure taken from them can be told from a stale one."""
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "elutq_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profile_figure(path, key):
    """`key: value` and `kernel source hash: ...` lines of a committed profile summary -> (value or None, hash matches)."""
    import re
    try:
        text = open(path).read()
    except OSError:
        return None, False
    m = re.search(r"^" + re.escape(key) + r":\s*([0-9.]+)", text, re.M)
    h = re.search(r"^kernel source hash:\s*([0-9a-f]+)", text, re.M)
    return (float(m.group(1)) if m else None), bool(h and h.group(1) == kernel_source_hash())
BITS, GROUP = 2, 128
N_LAYERS = 32


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    # default: a timed region of a few seconds per leg, long enough for a once-every-few-seconds GPU-busy sampler to see it
    p.add_argument("--steps", type=int, default=4000)
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline leg")
    p.add_argument("--no-decode", action="store_true", help="skip the decode tokens/s leg")
    p.add_argument("--no-gemm", action="store_true", help="skip the small-batch GEMM leg")
    p.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    p.add_argument("--sweep-only", action="store_true",
                   help="only the sweep and the per-shape rings of the per-GEMV entry point (no grouped / multi-stream / "
                        "copy / other-format / large-shape legs): the run a kernel trace of the dominant kernel is taken from")
    p.add_argument("--mode", choices=["full", "kernel", "copy", "decode", "decode-eager", "gemm", "group", "sparse"],
                   default="full",
                   help="kernel: only the dominant GEMV (4096x14336) over its weight ring, for counter runs; "
                        "copy: a plain 64 MiB device copy, the calibration kernel for FETCH_SIZE / WRITE_SIZE; "
                        "decode / gemm: only that leg (for kernel traces); "
                        "decode-eager: three eager decode steps of a two-layer model of the same widths (for counter runs); "
                        "sparse: GEMVs of layers with a block-sparse extra plane beside the same layers without it")
    p.add_argument("--launches", type=int, default=256, help="launches in --mode kernel / copy")
    return p.parse_args()


class Gemv:
    """Direct C-ABI launcher on preallocated buffers (no allocation in the timed loop)."""

    def __init__(self, lib, mod, x, y, ws):
        self.lib, self.mod, self.x, self.y, self.ws = lib, mod, x, y, ws
        self.args = (mod.planes.data_ptr(), mod.scales.data_ptr(), mod.zeros.data_ptr(), None,
                     x.data_ptr(), y.data_ptr(), mod.in_features, mod.out_features, mod.bits,
                     mod.group_size, ws.data_ptr(), ws.numel())

    def __call__(self, stream):
        rc = self.lib.elutq_hlq_gemv_f16(*self.args, stream)
        if rc:
            raise RuntimeError(f"elutq_hlq_gemv_f16 failed: {rc}")


def time_graph(torch, launch_all, replays, warmup, sustain_s=0.0, cold=None):
    """Captures launch_all(stream) once, replays it; returns seconds per replay (HIP events on
    the replay stream).  sustain_s > 0: after the `warmup` replays the graph is replayed untimed for that long, and
    the timed region is at least as long again, so that a leg whose rate follows the GPU's clocks is measured in the
    state a long run reaches (the clocks follow the load with a delay of tens of milliseconds) whatever `replays` is;
    the figure of the first `replays` replays after `warmup`, taken before that, goes into cold["s"]."""
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        launch_all(s.cuda_stream)            # eager warm-up on the capture stream
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        launch_all(torch.cuda.current_stream().cuda_stream)
    for _ in range(warmup):
        g.replay()
    torch.cuda.synchronize()

    def timed(n):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / n

    sec = timed(replays)
    if sustain_s <= 0:
        return sec
    if cold is not None:
        cold["s"] = sec
    n = max(replays, int(sustain_s / max(sec, 1e-7)) + 1)
    timed(n)                                 # untimed as far as the result goes
    return timed(n)


def cpu_baseline(budget_s):
    """C port of the reference CPU LUT GEMV (AVX2 pshufb lookups, fp32 accumulation) on the
    host cores: one layer's seven GEMVs, repeated within the time budget."""
    import numpy as np
    from elutq_amd.synth import LLAMA3_8B_SHAPES, algorithmic_bytes, make_layer
    from oracle import lutref
    if not os.path.exists(os.path.join(ROOT, "oracle", "liblutref.so")):
        lutref.build()
    ncpu = os.cpu_count() or 1
    out = {}
    weights = {}
    for (k, n) in sorted(set(LLAMA3_8B_SHAPES.values())):
        weights[(k, n)] = make_layer(k, n, bits=BITS, group=GROUP, seed=k + n)
    for threads in sorted({4, min(16, ncpu)}):
        refs = {kn: lutref.RefWeight(L.w_quant, L.w_scale, L.w_zero, GROUP, threads) for kn, L in weights.items()}
        seq = [(refs[kn], weights[kn].x[0]) for kn in LLAMA3_8B_SHAPES.values()]
        nbytes = sum(algorithmic_bytes(k, n, BITS, GROUP) for (k, n) in LLAMA3_8B_SHAPES.values())
        for rw, x in seq:
            rw.gemv_fast(x)
        t0 = time.perf_counter()
        reps = 0
        while True:
            for rw, x in seq:
                rw.gemv_fast(x)
            reps += 1
            if time.perf_counter() - t0 > budget_s / 2:
                break
        dt = (time.perf_counter() - t0) / reps
        out[threads] = {"GBps": nbytes / dt / 1e9, "ms_per_layer": dt * 1e3, "reps": reps}
    # the op-for-op restatement (every fp16 rounding of the reference chain, F16C conversions around each
    # operation; scalar inner loop) on the 4096 x 4096 projection, one thread and the reference's four
    kq = (4096, 4096)
    faithful = {}
    for threads in (1, 4):
        rw = lutref.RefWeight(weights[kq].w_quant, weights[kq].w_scale, weights[kq].w_zero, GROUP, threads)
        rw.gemv(weights[kq].x[0])
        t0, reps = time.perf_counter(), 0
        while reps < 3 or time.perf_counter() - t0 < 1.0:
            rw.gemv(weights[kq].x[0])
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        faithful[threads] = {"GBps": algorithmic_bytes(*kq, BITS, GROUP) / dt / 1e9, "ms_per_gemv": dt * 1e3, "reps": reps}
    out["fp16_faithful_4096x4096"] = faithful
    return out, ncpu


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


MFMA_PEAK_TFLOPS = 2500.0      # dense fp16 / bf16


def gemm_leg(torch, lib, dev, steps):
    """Small-batch GEMM, HLQ w2g128, M in {16, 32, 64}, LLaMA-2-13B shapes;
    each over a ring of weight sets > 400 MB.  Reports both roofline fractions (MFMA and HBM)."""
    from elutq_amd.synth import LLAMA2_13B_PREFILL_SHAPES, algorithmic_bytes, make_device_layer
    out = {}
    for (k, n) in LLAMA2_13B_PREFILL_SHAPES:
        nsets = -(-400 * 2 ** 20 // algorithmic_bytes(k, n, BITS, GROUP, 16))
        mods = [make_device_layer(k, n, BITS, GROUP, seed=50_000 + i, device=dev) for i in range(nsets)]
        for m in (16, 32, 64):
            x = torch.randn(m, k, device=dev).to(torch.float16)
            y = torch.empty(m, n, dtype=torch.float16, device=dev)
            ws = torch.zeros(lib.elutq_hlq_workspace_bytes(k, n, BITS, GROUP, m), dtype=torch.uint8, device=dev)

            def launch(stream):
                for md in mods:
                    rc = lib.elutq_hlq_gemm_f16(md.planes.data_ptr(), md.scales.data_ptr(), md.zeros.data_ptr(), None,
                                                x.data_ptr(), y.data_ptr(), m, k, n, BITS, GROUP, ws.data_ptr(),
                                                ws.numel(), stream)
                    if rc:
                        raise RuntimeError(f"elutq_hlq_gemm_f16 failed: {rc}")

            sec = time_graph(torch, launch, max(3, min(steps, 200)), 2) / nsets
            flops, nbytes = 2.0 * m * k * n, algorithmic_bytes(k, n, BITS, GROUP, m)
            out[f"{k}x{n}_M{m}"] = {"us": sec * 1e6, "TFLOPs": flops / sec / 1e12,
                                    "frac_mfma_peak": flops / sec / 1e12 / MFMA_PEAK_TFLOPS,
                                    "GBps": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}
        del mods
        torch.cuda.empty_cache()
    return out


def sparse_leg(torch, lib, dev, steps, warmup, density=0.1, ring_len=16):
    """Batch-1 GEMV of w2g128 layers that carry a block-sparse extra plane on `density` of their
    (32 channels x 128 inputs) blocks, held as blocks: looked up inside the dense launch (the inline form) and as
    two launches (the plane's fp32 term, then the dense GEMV that adds it), next to the same dense layers alone and to
    layers of one more dense plane (the form the loader gives the plane by default).  Weight rings of `ring_len`
    layers per shape."""
    import numpy as np

    from elutq_amd.hlq_linear import sparse_index
    from elutq_amd.synth import LLAMA3_8B_SHAPES, algorithmic_bytes, make_device_layer
    out = {}
    for name in ("q_proj", "gate_proj"):
        k, n = LLAMA3_8B_SHAPES[name]
        g = torch.Generator().manual_seed(k + n)
        pick = (torch.rand(n // 32, k // GROUP, generator=g) < density).nonzero()
        mask = torch.stack([pick[:, 0] * 32, pick[:, 1] * GROUP], 1).numpy().astype(np.uint32)
        nblk = mask.shape[0]
        index = torch.from_numpy(sparse_index(mask, k, n, GROUP)).to(dev)
        ring = []
        for i in range(ring_len):
            mod = make_device_layer(k, n, BITS, GROUP, seed=i, device=dev)
            blocks = torch.randint(0, 256, (nblk, 32, GROUP // 8), dtype=torch.uint8, device=dev)
            scales = (torch.rand(nblk, 32, device=dev) * 0.06 + 0.02).to(torch.float16)
            ring.append((mod, blocks, scales))
        x = torch.randn(1, k, device=dev).to(torch.float16)
        y = torch.empty(1, n, dtype=torch.float16, device=dev)
        ws = torch.zeros(lib.elutq_hlq_sparse_workspace_bytes(k, n, BITS, GROUP, 1), dtype=torch.uint8, device=dev)

        def launch_sparse(stream):
            for mod, blocks, scales in ring:
                rc = lib.elutq_hlq_sparse_gemv_f16(mod.planes.data_ptr(), mod.scales.data_ptr(), mod.zeros.data_ptr(), None,
                                                   blocks.data_ptr(), scales.data_ptr(), index.data_ptr(), nblk,
                                                   x.data_ptr(), y.data_ptr(), k, n, BITS, GROUP, ws.data_ptr(), ws.numel(), stream)
                if rc:
                    raise RuntimeError(f"elutq_hlq_sparse_gemv_f16 failed: {rc}")

        dense = [Gemv(lib, mod, x, y, ws) for mod, _, _ in ring]

        def launch_dense(stream):
            for gv in dense:
                gv(stream)

        t_sp = time_graph(torch, launch_sparse, steps, warmup) / ring_len
        t_de = time_graph(torch, launch_dense, steps, warmup) / ring_len
        # inside a decode step: RMSNorm in front of the projection (formed by both launches), residual behind
        from elutq_amd.hlq_linear import HLQLinear
        fused = [HLQLinear(k, n, BITS, GROUP, mod.planes, mod.scales, mod.zeros, None, (blocks, scales, index))
                 for mod, blocks, scales in ring]
        norm_w = torch.ones(k, dtype=torch.float16, device=dev)
        res = torch.randn(1, n, device=dev).to(torch.float16)

        def launch_fused(stream, mods=fused):       # (time_graph makes `stream` the current one)
            for m in mods:
                m.gemv_fused(x, y, ws, prologue=1, norm_weight=norm_w, eps=1e-5, residual=res)

        def launch_fused_dense(stream):
            launch_fused(stream, [mod for mod, _, _ in ring])

        def launch_inline(stream):                  # plain call, the blocks looked up inside the dense launch
            for m in fused:
                m.gemv_fused(x, y, ws)

        assert all(m.sparse_inline is not None for m in fused)
        t_in = time_graph(torch, launch_inline, steps, warmup) / ring_len
        t_fi = time_graph(torch, launch_fused, steps, warmup) / ring_len
        HLQLinear.use_sparse_inline = False         # the plane as a launch of its own in front of the dense one
        try:
            t_fu = time_graph(torch, launch_fused, steps, warmup) / ring_len
        finally:
            HLQLinear.use_sparse_inline = True
        t_fd = time_graph(torch, launch_fused_dense, steps, warmup) / ring_len
        # the plane written out as one more dense plane (scale 0 where no block exists): what the loader does
        # by default -- it costs what any layer with one more plane costs
        wide = [Gemv(lib, make_device_layer(k, n, BITS + 1, GROUP, seed=100 + i, device=dev), x, y, ws) for i in range(ring_len)]

        def launch_wide(stream):
            for gv in wide:
                gv(stream)

        t_wi = time_graph(torch, launch_wide, steps, warmup) / ring_len
        sparse_bytes = nblk * (32 * GROUP // 8 + 64 + 4) + 4 * (n // 32 + 1) + 8 * n      # blocks, scales, index, fp32 term out and in
        out[f"{k}x{n}"] = {"blocks": nblk, "density": density, "inline_layer_us": t_in * 1e6, "two_launch_layer_us": t_sp * 1e6,
                           "dense_layer_us": t_de * 1e6, "as_one_more_dense_plane_us": t_wi * 1e6,
                           "rmsnorm_residual_inline_layer_us": t_fi * 1e6, "rmsnorm_residual_two_launch_layer_us": t_fu * 1e6,
                           "rmsnorm_residual_dense_layer_us": t_fd * 1e6,
                           "sparse_plane_bytes": sparse_bytes, "dense_bytes": algorithmic_bytes(k, n, BITS, GROUP)}
    out["decode"] = sparse_decode_leg(torch, dev, density)
    return out


def sparse_decode_leg(torch, dev, density, n_ctx=512, n_gen=50):
    """Decode tokens/s of the LLaMA-3-8B-shaped w2g128 model whose every projection carries a sparse extra plane on
    `density` of its blocks, held as blocks and looked up inside the projections' own launches."""
    from elutq_amd.llama_decode import LlamaDecoder, LlamaShape, random_parts
    from elutq_amd.synth import with_device_sparse_plane
    s = LlamaShape()
    parts = random_parts(s, dev, 0)
    seed, nblk = 1, 0
    for lin, _ in parts["layers"]:
        for name in list(lin):
            lin[name] = with_device_sparse_plane(lin[name], density, seed)
            nblk += lin[name].sparse_count
            seed += 1
    model = LlamaDecoder(s, device=dev, seed=0, parts=parts)
    model.fill_cache(n_ctx)
    model.token.fill_(1)
    model.capture()
    for _ in range(n_gen):                       # untimed pass over the same tokens, then the timed one
        model.replay()
    model.pos.fill_(n_ctx)
    model.token.fill_(1)
    model.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_gen - 1):
        model.replay()
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    return {"tokens_per_s": (n_gen - 1) / sec, "ms_per_token": sec / (n_gen - 1) * 1e3, "blocks": nblk, "density": density,
            "model": "LLaMA-3-8B-shaped random init, 32 layers, HLQ w2g128 + sparse extra plane held as blocks on every "
                     "projection (inline form: one launch per projection), fp16 lm_head", "n_ctx": n_ctx, "n_gen": n_gen}


def counter_mode(a, torch, lib, dev):
    """Eager launches of one kernel only, so a rocprofv3 --pmc run sees nothing else of size."""
    from elutq_amd.synth import algorithmic_bytes, make_device_layer
    if a.mode == "copy":
        n = 64 * 2 ** 20
        src = torch.randint(0, 255, (n,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(a.launches):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"mode": "copy", "bytes_read": n, "bytes_written": n, "launches": a.launches}))
        return
    k, n = 4096, 14336
    nbytes = algorithmic_bytes(k, n, BITS, GROUP)
    ring = [make_device_layer(k, n, BITS, GROUP, seed=i, device=dev) for i in range(-(-512 * 2 ** 20 // nbytes))]
    x = torch.randn(1, k, device=dev).to(torch.float16)
    y = torch.empty(1, n, dtype=torch.float16, device=dev)
    ws = torch.zeros(lib.elutq_hlq_workspace_bytes(k, n, BITS, GROUP, 1), dtype=torch.uint8, device=dev)
    calls = [Gemv(lib, m, x, y, ws) for m in ring]
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    for i in range(a.launches):
        calls[i % len(calls)](stream)
    torch.cuda.synchronize()
    print(json.dumps({"mode": "kernel", "shape": f"{k}x{n}", "algorithmic_bytes": nbytes, "launches": a.launches,
                      "ring_sets": len(ring)}))


SUSTAIN_S = 0.08       # untimed lead of the legs whose rate follows the GPU's clocks (and the least length of their timed region)


def side_legs(a, torch, lib, dev, calls, xs, ws_bytes, step_bytes):
    """The same 224 GEMVs through the grouped entry point (one launch on the engine the library picks -- the streaming
    matrix-core kernel -- and on the LUT engine; one launch per layer), the per-GEMV launches dealt onto four streams
    of one graph, and a plain device copy as a yardstick."""
    from elutq_amd import _lib
    from elutq_amd.hlq_linear import GemvGroup
    from elutq_amd.synth import LLAMA3_8B_SHAPES
    g_mods = [c.mod for c in calls]
    g_xs = [xs[m.in_features] for m in g_mods]
    g_ys = [torch.empty(1, m.out_features, dtype=torch.float16, device=dev) for m in g_mods]
    grouped = {}
    engine_before = lib.elutq_hlq_get_gemv_engine()
    for label, per, engine in (("one_launch", len(g_mods), None), ("one_launch_lut_engine", len(g_mods), "lut"),
                               ("launch_per_layer", len(LLAMA3_8B_SHAPES), None)):
        if engine:
            _lib.set_gemv_engine(engine)
        groups = [GemvGroup(g_mods[i:i + per], g_xs[i:i + per], g_ys[i:i + per]) for i in range(0, len(g_mods), per)]
        lib.elutq_hlq_set_gemv_engine(engine_before)

        def launch_groups(stream, groups=groups):
            for g in groups:
                g.run()

        cold = {}
        sec = time_graph(torch, launch_groups, a.steps, a.warmup, SUSTAIN_S, cold)
        grouped[label] = {"launches": len(groups), "ms_per_step": sec * 1e3, "GBps": step_bytes / sec / 1e9,
                          "frac_hbm_peak": step_bytes / sec / 1e9 / HBM_PEAK_GBPS,
                          # the first `steps` replays after `warmup`, before the clocks have followed the load
                          "cold_GBps": step_bytes / cold["s"] / 1e9, "sustained_lead_s": SUSTAIN_S}
        for g in groups:
            g.close()
    grouped["one_launch"]["kernel"] = ("hlq_gemv_mfma_group_kernel<2,false>: fp4 x fp4 MFMA on the plane bits, 256 workgroups, "
                                       "each streaming one contiguous share of the 2.08 GB")
    grouped["one_launch"]["roofline"] = {"bound": "hbm", "achieved": grouped["one_launch"]["GBps"], "peak": HBM_PEAK_GBPS,
                                         "unit": "GB/s", "frac": grouped["one_launch"]["frac_hbm_peak"],
                                         "bytes_per_launch": step_bytes}
    # ---- the same 224 launches of the per-GEMV entry point, dealt round-robin onto four HIP streams
    # inside one graph (a workspace per stream): independent GEMVs overlap each other's start-up and tail
    n_streams = 4
    c_ws = [torch.zeros(ws_bytes, dtype=torch.uint8, device=dev) for _ in range(n_streams)]
    c_calls = [Gemv(lib, m, g_xs[i], g_ys[i], c_ws[i % n_streams]) for i, m in enumerate(g_mods)]
    side = [torch.cuda.Stream() for _ in range(n_streams - 1)]

    def launch_concurrent(stream):
        main = torch.cuda.current_stream()
        fork = torch.cuda.Event()
        fork.record(main)
        for s in side:
            s.wait_event(fork)
        handles = [stream] + [s.cuda_stream for s in side]
        for i, c in enumerate(c_calls):
            c(handles[i % n_streams])
        for s in side:
            join = torch.cuda.Event()
            join.record(s)
            main.wait_event(join)

    sec = time_graph(torch, launch_concurrent, a.steps, a.warmup)
    grouped["per_gemv_launches_on_4_streams"] = {"launches": len(c_calls), "streams": n_streams, "ms_per_step": sec * 1e3,
                                                 "GBps": step_bytes / sec / 1e9,
                                                 "frac_hbm_peak": step_bytes / sec / 1e9 / HBM_PEAK_GBPS}
    del g_ys, c_calls, c_ws, side
    # what a plain device-to-device copy reaches on this GPU (read + write bytes), as a yardstick
    cp_a = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    cp_b = torch.empty_like(cp_a)
    sec = time_graph(torch, lambda s: cp_b.copy_(cp_a), 10, 2)
    grouped["device_copy_1GiB_GBps"] = 2 * cp_a.numel() / sec / 1e9
    del cp_a, cp_b
    torch.cuda.empty_cache()

    return grouped


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py: this build measures ONE GPU (the path needs no collective); --gpus {a.gpus} is not supported",
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from elutq_amd import _lib
    from elutq_amd.synth import LLAMA3_8B_SHAPES, algorithmic_bytes, make_device_layer

    lib = _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if a.mode == "decode":
        from elutq_amd.llama_decode import bench_decode
        print(json.dumps({"mode": "decode", "decode": bench_decode(dev),
                          "decode_hlq_lm_head": bench_decode(dev, hlq_lm_head=True)}))
        return
    if a.mode == "decode-eager":
        # a reduced decode for counter runs (rocprofv3 --pmc serialises every dispatch, and the full 32-layer graph
        # replay does not finish under it): two layers of the LLaMA-3-8B widths, three eager steps, no graph
        from elutq_amd.hlq_linear import HLQLinear
        from elutq_amd.llama_decode import LlamaDecoder, LlamaShape
        shape = LlamaShape(n_layers=2)
        model = LlamaDecoder(shape, device=dev, seed=0)
        model.fill_cache(512)
        model.token.fill_(1)
        steps = 3
        for _ in range(steps):
            model.step()
        torch.cuda.synchronize()
        hlq_bytes = sum(m.planes.numel() + m.scales.numel() + m.zeros.numel() for m in model.modules() if isinstance(m, HLQLinear))
        kv_bytes = 2 * shape.n_layers * 512 * shape.n_kv_heads * shape.head_dim * 2
        print(json.dumps({"mode": "decode-eager", "layers": shape.n_layers, "steps": steps,
                          "algorithmic_bytes_per_step": {"hlq_layers": hlq_bytes, "fp16_lm_head": model.lm_head.numel() * 2,
                                                         "kv_cache_read": kv_bytes, "embedding_row": shape.hidden * 2}}))
        return
    if a.mode == "gemm":
        print(json.dumps({"mode": "gemm", "gemm_w2g128_llama2_13b": gemm_leg(torch, lib, dev, a.steps)}))
        return
    if a.mode == "group":
        # the whole sweep as one grouped launch, `steps` times (for rocprofv3 --kernel-trace)
        from elutq_amd.hlq_linear import GemvGroup
        mods, nbytes = [], 0
        for i in range(N_LAYERS):
            for (k, n) in LLAMA3_8B_SHAPES.values():
                mods.append(make_device_layer(k, n, BITS, GROUP, seed=len(mods), device=dev))
                nbytes += algorithmic_bytes(k, n, BITS, GROUP)
        xk = {k: torch.randn(1, k, device=dev).to(torch.float16) for k in {m.in_features for m in mods}}
        grp = GemvGroup(mods, [xk[m.in_features] for m in mods],
                        [torch.empty(1, m.out_features, dtype=torch.float16, device=dev) for m in mods])
        cold = {}
        sec = time_graph(torch, lambda s: grp.run(), a.steps, a.warmup, SUSTAIN_S, cold)
        print(json.dumps({"mode": "group", "gemvs_per_launch": len(mods), "bytes_per_launch": nbytes, "us_per_launch": sec * 1e6,
                          "GBps": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                          "cold_GBps": nbytes / cold["s"] / 1e9, "engine": lib.elutq_hlq_get_gemv_engine()}))
        grp.close()
        return
    if a.mode == "sparse":
        print(json.dumps({"mode": "sparse", "sparse_gemv_w2g128": sparse_leg(torch, lib, dev, a.steps, a.warmup)}))
        return
    if a.mode != "full":
        counter_mode(a, torch, lib, dev)
        return
    ws_bytes = max(lib.elutq_hlq_workspace_bytes(k, n, BITS, GROUP, 1) for (k, n) in LLAMA3_8B_SHAPES.values())
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
    xs = {k: torch.randn(1, k, device=dev).to(torch.float16) for k in {k for k, _ in LLAMA3_8B_SHAPES.values()}}
    ys = {n: torch.empty(1, n, dtype=torch.float16, device=dev) for n in {n for _, n in LLAMA3_8B_SHAPES.values()}}

    # ---- the sweep: 32 layers x 7 projections, all weight sets distinct -----------------
    calls = []
    step_bytes = 0
    seed = 0
    for layer in range(N_LAYERS):
        for name, (k, n) in LLAMA3_8B_SHAPES.items():
            mod = make_device_layer(k, n, BITS, GROUP, seed=seed, device=dev)
            seed += 1
            calls.append(Gemv(lib, mod, xs[k], ys[n], ws))
            step_bytes += algorithmic_bytes(k, n, BITS, GROUP)
    torch.cuda.synchronize()

    def launch_step(stream):
        for c in calls:
            c(stream)

    sec_step = time_graph(torch, launch_step, a.steps, a.warmup)
    value = step_bytes / sec_step / 1e9

    grouped = {}
    if not a.sweep_only:
        grouped = side_legs(a, torch, lib, dev, calls, xs, ws_bytes, step_bytes)

    # ---- per shape, each over a ring of weight sets > 512 MB ------------------------------
    per_shape = {}
    by_shape = {}
    for c in calls:
        by_shape.setdefault((c.mod.in_features, c.mod.out_features), []).append(c)
    for (k, n), lst in sorted(by_shape.items()):
        nbytes = algorithmic_bytes(k, n, BITS, GROUP)
        need = -(-512 * 2 ** 20 // nbytes)
        extra = []
        while len(lst) + len(extra) < need:
            mod = make_device_layer(k, n, BITS, GROUP, seed=10_000 + len(extra) + k, device=dev)
            extra.append(Gemv(lib, mod, xs[k], ys[n], ws))
        ring = lst + extra

        def launch_ring(stream, ring=ring):
            for c in ring:
                c(stream)

        reps = max(3, min(a.steps, int(20000 / len(ring)) + 1))
        sec = time_graph(torch, launch_ring, reps, 2) / len(ring)
        # the same GEMV over ONE weight set, launched 64 times per replay: the weights then stay in
        # the 256 MB last-level cache, so this is the kernel without its HBM stream
        hot = lst[0]

        def launch_hot(stream, hot=hot):
            for _ in range(64):
                hot(stream)

        sec_hot = time_graph(torch, launch_hot, max(3, min(a.steps, 500)), 2) / 64
        per_shape[f"{k}x{n}"] = {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                                 "bytes": nbytes, "ring_sets": len(ring),
                                 "cache_resident_us": sec_hot * 1e6, "cache_resident_GBps": nbytes / sec_hot / 1e9}
        del extra, ring
        torch.cuda.empty_cache()

    # ---- the same four shapes at w3g128 and w2g64 (plane count and group size in the fold) ---
    other_formats = {}
    for bits, group in (() if a.sweep_only else ((3, 128), (2, 64))):
        res = {}
        for (k, n) in sorted(set(LLAMA3_8B_SHAPES.values())):
            nbytes = algorithmic_bytes(k, n, bits, group)
            ring = []
            for i in range(-(-512 * 2 ** 20 // nbytes)):
                mod = make_device_layer(k, n, bits, group, seed=20_000 + i + k, device=dev)
                ring.append(Gemv(lib, mod, xs[k], ys[n], ws))

            def launch_ring(stream, ring=ring):
                for c in ring:
                    c(stream)

            reps = max(3, min(a.steps, int(20000 / len(ring)) + 1))
            sec = time_graph(torch, launch_ring, reps, 2) / len(ring)
            res[f"{k}x{n}"] = {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                               "bytes": nbytes}
            del ring
            torch.cuda.empty_cache()
        other_formats[f"w{bits}g{group}"] = res

    large_shape = {}
    if not a.sweep_only:
        # ---- one GEMV large enough that the launch and its start-up no longer matter: an lm_head-sized
        # layer (vocabulary 128256) at w2g128, over a ring of distinct weight sets
        k, n = 4096, 128256
        nbytes = algorithmic_bytes(k, n, BITS, GROUP)
        ring = [Gemv(lib, make_device_layer(k, n, BITS, GROUP, seed=30_000 + i, device=dev), xs[k],
                     torch.empty(1, n, dtype=torch.float16, device=dev), ws) for i in range(4)]

        def launch_big(stream, ring=ring):
            for c in ring:
                c(stream)

        cold = {}
        sec = time_graph(torch, launch_big, max(3, min(a.steps, 2000)), 5, SUSTAIN_S, cold) / len(ring)
        large_shape = {f"{k}x{n}": {"us": sec * 1e6, "GBps": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                                    "bytes": nbytes, "ring_sets": len(ring), "cold_us": cold["s"] / len(ring) * 1e6}}
        # ---- a wide layer with K > 4096 (a 14336 x 32768 projection, 143 MB): here the library's choice is the streaming
        # matrix-core kernel (no K slices), beside the LUT kernel's runs of column blocks with K slices
        from elutq_amd import _lib as _l
        k2, n2 = 14336, 32768
        nbytes2 = algorithmic_bytes(k2, n2, BITS, GROUP)
        ws2 = torch.zeros(lib.elutq_hlq_workspace_bytes(k2, n2, BITS, GROUP, 1), dtype=torch.uint8, device=dev)
        ring2 = [Gemv(lib, make_device_layer(k2, n2, BITS, GROUP, seed=31_000 + i, device=dev), xs[k2],
                      torch.empty(1, n2, dtype=torch.float16, device=dev), ws2) for i in range(4)]

        def launch_big2(stream):
            for c in ring2:
                c(stream)

        sec = time_graph(torch, launch_big2, max(3, min(a.steps, 2000)), 5, SUSTAIN_S) / len(ring2)
        engine_before = lib.elutq_hlq_get_gemv_engine()
        _l.set_gemv_engine("lut")
        sec_lut = time_graph(torch, launch_big2, max(3, min(a.steps, 2000)), 5, SUSTAIN_S) / len(ring2)
        lib.elutq_hlq_set_gemv_engine(engine_before)
        large_shape[f"{k2}x{n2}"] = {"us": sec * 1e6, "GBps": nbytes2 / sec / 1e9, "frac_hbm_peak": nbytes2 / sec / 1e9 / HBM_PEAK_GBPS,
                                     "bytes": nbytes2, "ring_sets": len(ring2), "lut_engine_us": sec_lut * 1e6}
        del ring2, ws2
        torch.cuda.empty_cache()
        # ---- the same lm_head unquantized: the dense fp16 GEMV of the decode step (two weight sets of 1.05 GB),
        # beside the hipBLASLt call it replaced
        wsets = [(torch.randn(n, k, device=dev) * 0.02).to(torch.float16) for _ in range(2)]
        yb = torch.empty(1, n, dtype=torch.float16, device=dev)

        def launch_dense(stream):
            for w in wsets:
                rc = lib.elutq_fp16_gemv_f16(w.data_ptr(), None, xs[k].data_ptr(), yb.data_ptr(), k, n, None, 0.0, stream)
                if rc:
                    raise RuntimeError(f"elutq_fp16_gemv_f16 failed: {rc}")

        def launch_blas(stream):
            for w in wsets:
                torch.mm(xs[k], w.t(), out=yb)

        fbytes = 2 * n * k + 2 * k + 2 * n
        sec = time_graph(torch, launch_dense, max(3, min(a.steps, 1000)), 5) / len(wsets)
        secb = time_graph(torch, launch_blas, max(3, min(a.steps, 1000)), 5) / len(wsets)
        large_shape[f"fp16_{k}x{n}"] = {"us": sec * 1e6, "GBps": fbytes / sec / 1e9, "frac_hbm_peak": fbytes / sec / 1e9 / HBM_PEAK_GBPS,
                                        "bytes": fbytes, "ring_sets": len(wsets), "hipblaslt_us": secb * 1e6}
        del wsets
        torch.cuda.empty_cache()

    dom = per_shape["4096x14336"]
    # HBM bytes per launch of this kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --mode kernel`,
    # each scaled by what the same counter reads for `--mode copy`: read from the committed summary, a property of the
    # kernel's access pattern, not of this run -- and null when the kernel's sources are no longer the ones measured
    traffic, traffic_fresh = profile_figure(TRAFFIC_PROFILE, "traffic bytes per launch")
    trace_us, trace_fresh = profile_figure(TRACE_PROFILE, "average duration us")
    roofline = {"bound": "hbm", "achieved": dom["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": dom["GBps"] / HBM_PEAK_GBPS,
                "traffic": int(traffic) if traffic and traffic_fresh else None,
                "traffic_source": "profiles/hlq_gemv_w2g128_4096x14336_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE of "
                                  "`bench.py --mode kernel`, scaled by the same counters of `--mode copy`), not measured in this run"
                                  + ("" if traffic_fresh else "; the kernel's sources have changed since that measurement, so no figure is quoted"),
                "kernel": "hlq_gemv_kernel<2,false> K=4096 N=14336", "us_per_launch": dom["us"],
                "bytes_per_launch": dom["bytes"], "kernel_source_hash": kernel_source_hash()}
    if trace_us and trace_fresh:
        # the same kernel's average start-to-end duration in the rocprofv3 kernel trace of `bench.py --sweep-only`
        # (profiles/hlq_gemv_w2g128_sweep_kernel_trace.md) and the fraction that follows from it: a replayed launch
        # starts while its predecessor's completion is still being signalled, so the live per-launch period above
        # is shorter than the traced duration
        roofline["kernel_trace_avg_us"] = trace_us
        roofline["frac_kernel_trace"] = dom["bytes"] / (trace_us * 1e-6) / 1e9 / HBM_PEAK_GBPS
    if grouped.get("device_copy_1GiB_GBps"):
        roofline["frac_of_device_copy_rate"] = dom["GBps"] / grouped["device_copy_1GiB_GBps"]

    out = {
        "metric": "LUT-GEMV HBM GB/s at LLaMA3-8B shapes bs1 (HLQ w2g128)",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": sec_step * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16 activations, int32 fixed-point tables, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "LLaMA-3-8B layer-shape sweep, HLQ w2g128, batch 1: 32 layers x (q,k,v,o,gate,up,down) = 224 GEMVs over distinct weights per step",
                   "bits": BITS, "group": GROUP, "bytes_per_step": step_bytes, "gemvs_per_step": len(calls)},
        "frac_hbm_peak": value / HBM_PEAK_GBPS,
        "per_shape": per_shape,
        "per_shape_other_formats": other_formats,
        "large_shape": large_shape,
        "roofline": roofline,
        # supplementary: the same 224 GEMVs handed to elutq_hlq_gemv_group_* (they are independent in this
        # sweep); `value` above stays the one-call-per-GEMV figure of the drop-in entry point
        "grouped_sweep": grouped,
    }

    if not a.no_gemm:
        out["gemm_w2g128_llama2_13b"] = gemm_leg(torch, lib, dev, a.steps)

    if not a.no_decode:
        try:
            from elutq_amd.llama_decode import bench_decode
            out["decode"] = bench_decode(dev)
            # the same model with the lm_head quantized like every other layer, which is what the
            # reference's exporter writes unless it is told to skip the lm_head (extra information:
            # the workload of the headline decode figure keeps the fp16 lm_head)
            torch.cuda.empty_cache()
            out["decode_hlq_lm_head"] = bench_decode(dev, hlq_lm_head=True)
            # the same step (fp16 lm_head) at the other formats of the GEMV sweep
            from elutq_amd.llama_decode import LlamaShape
            out["decode_other_formats"] = {}
            for bits, group in ((3, 128), (2, 64)):
                torch.cuda.empty_cache()
                r = bench_decode(dev, shape=LlamaShape(bits=bits, group=group))
                out["decode_other_formats"][f"w{bits}g{group}"] = {k: r[k] for k in ("tokens_per_s", "ms_per_token",
                                                                                     "bytes_per_token", "GBps")}
        except ImportError:
            out["decode"] = None

    if not a.no_cpu:
        res, ncpu = cpu_baseline(a.cpu_seconds)
        faithful = res.pop("fp16_faithful_4096x4096")
        tmax = max(res)
        out["cpu_baseline"] = {"value": res[tmax]["GBps"], "unit": "GB/s", "cores": tmax, "kind": "port",
                               "sample": f"one layer (7 GEMVs, {res[tmax]['reps']} repeats) of the same sweep, AVX2 port of the reference kernel with fp32 accumulators, {tmax} OpenMP threads of {ncpu} host CPUs",
                               "ms_per_layer": res[tmax]["ms_per_layer"],
                               "at_4_threads_GBps": res[4]["GBps"] if 4 in res else None,
                               "cpu_model": cpu_model(), "host_cpus": ncpu,
                               "fp16": "fp16 storage, F16C conversions, fp32 accumulate (the port); the reference's NEON kernel "
                                       "accumulates in fp16, restated op for op below",
                               "fp16_faithful_scalar_4096x4096": faithful}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
