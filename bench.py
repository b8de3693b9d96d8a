#!/usr/bin/env python3
"""Benchmark of the GGUF quantised-matmul hot path on one MI355X.

Headline (`value`): the Q4_K decode GEMV at K=4096, N=14336, batch 1, as algorithmic HBM GB/s.
One "step" is one GEMV launch.  The steps rotate over distinct weight buffers (> 512 MB in
total) so every launch streams its 33 MB from HBM rather than from the 256 MB last-level cache.
The same JSON line carries
  * `roofline`: that kernel against the 8 TB/s HBM peak;
  * `cpu_baseline`: the CPU checker's restatement of the reference path timed on this host (one
    thread; with the Interpreter's weight copy; the one-off dequantisation; an all-cores form
    that is not the reference);
  * `gemv_configs`: the Q8_0 4096 x 4096 and the Q4_0 / Q4_K FFN-shape GEMVs, each with a roofline;
  * `prefill_gemm`: the matrix-core GEMM at M = 16 / 64 / 512;
  * `decode`: greedy decode of the random-init 7B-shape Q4_0 model (prompt 128, 256 new tokens),
    with the CPU checker's tokens per second beside it;
  * `decode_8b`: the 8B GQA shape with mixed Q4_K / Q6_K weights, prompt 512 + 512 tokens at
    context 4096;
  * with --microbench, `microbench`: an empty kernel, a read-only kernel, the GEMV's in-kernel
    timeline, the matrix-core GEMM's instruction mix, what a meeting of the workgroups of one XCD
    costs inside a launch, and the decoder-block kernel's in-kernel timeline.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-decode] [--no-cpu] [--no-gemm]
       [--no-configs] [--microbench]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "gemv_q4_k_14336x4096_hbm_traffic.txt")
CONFIG_TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "gemv_configs_hbm_traffic.txt")


def measured_traffic_bytes():
    """HBM bytes one launch of the headline GEMV moves, as the committed profiler summary states
    them (rocprofv3 FETCH_SIZE / WRITE_SIZE scaled by a known-size copy); a property of the kernel
    and the shape, not re-measured by this script.  None when the summary is not there."""
    import re
    try:
        with open(TRAFFIC_SUMMARY) as f:
            m = re.search(r"GEMV traffic per launch:.*= (\d+) bytes", f.read())
        return int(m.group(1)) if m else None
    except OSError:
        return None


def traffic_source():
    """Where `roofline.traffic` comes from: the committed summary and the commit that last touched it."""
    import subprocess
    rel = os.path.relpath(TRAFFIC_SUMMARY, ROOT)
    try:
        rev = subprocess.run(["git", "-C", ROOT, "log", "-1", "--format=%h", "--", rel], capture_output=True, text=True,
                             timeout=10).stdout.strip()
    except (OSError, subprocess.SubprocessError):
        rev = ""
    try:
        import hashlib
        with open(TRAFFIC_SUMMARY, "rb") as f:
            digest = hashlib.sha256(f.read()).hexdigest()[:16]
    except OSError:
        digest = None
    # the commit is known only where the git history is at hand; the digest names the file's
    # contents everywhere (sha256sum <file> | cut -c1-16)
    return {"file": rel, "commit": rev or None, "sha256_16": digest,
            "note": "a property of the kernel and the shape, measured with rocprofv3 --pmc when the kernel last "
                    "changed; not re-measured by this run"}


def last_gemm_launch():
    """The instance and grid of the matrix-core kernel this thread launched last, as the library reports it."""
    import ctypes as C
    from litenn_amd._lib import check, load
    buf = C.create_string_buffer(256)
    check(load().litenn_hip_gemm_last_launch(buf, len(buf)))
    return buf.value.decode()


def last_gemv_launch():
    """The instance and geometry of the streaming kernel this thread launched last, as the library reports it."""
    import ctypes as C
    from litenn_amd._lib import check, load
    buf = C.create_string_buffer(512)
    check(load().litenn_hip_gemv_last_launch(buf, len(buf)))
    return buf.value.decode()


def measured_config_traffic():
    """{(format name, n, k): HBM bytes per launch} of the other single-row configurations, from their
    committed profiler summary (same method as the headline's); empty when the summary is not there."""
    import re
    out = {}
    try:
        with open(CONFIG_TRAFFIC_SUMMARY) as f:
            for m in re.finditer(r"^(Q\w+) GEMV (\d+)x(\d+) traffic per launch:.*= (\d+) bytes", f.read(), re.M):
                out[(m.group(1), int(m.group(2)), int(m.group(3)))] = int(m.group(4))
    except OSError:
        pass
    return out


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def bench_gemv(ln, hiprt, fmt, n, k, steps, warmup, n_buffers, seed=1, graph_rotations=16):
    """Times `steps` launches of the GEMV rotating over `n_buffers` weight buffers.
    Returns (ms_per_step from HIP events on the launch stream, wall ms per step)."""
    from litenn_amd import synth
    from litenn_amd._lib import Exec, check, load
    import ctypes as C

    lib = load()
    wq_host = synth.quant_weights(fmt, n, k, seed)
    weights = []
    for b in range(n_buffers):
        # distinct memory, distinct contents (rolled rows) without regenerating 33 MB each time
        weights.append(ln.Tensor.from_numpy(np.roll(wq_host, b, axis=0).reshape(-1)))
    x = ln.Tensor.from_numpy(synth.activations(1, k, seed + 1))
    y = ln.Tensor((1, n))
    stream = hiprt.Stream()
    opts = Exec(stream.handle, 0)

    def launch(i):
        check(lib.litenn_hip_mul_mat_q(0, fmt, weights[i % n_buffers].ptr, n, k, x.ptr, 0, 1, y.ptr, None, 0,
                                       C.byref(opts)))

    for i in range(warmup):
        launch(i)
    stream.synchronize()
    # The launches are captured as graphs so that the host stays out of the timed region.  Starting a
    # graph costs about 13 us on the device whatever it holds (measured with empty kernels: 14.4 us
    # for a graph of one, 1.58 us per kernel in a graph of 256, 1.53 us per kernel launched
    # directly), so a graph holds up to 16 rotations; exactly `steps` kernels run, all from graphs.
    # A short run (fewer than 64 steps) times a graph of exactly `steps` launches between two events
    # in the middle of a busy queue: SHORT_RUN_PRIMING replays of a graph of 256 launches go first
    # (about 16 ms: the card is then at the clocks it sustains, and the queue never runs dry), and
    # nothing synchronises before the timed graph.  The region is taken SHORT_RUN_REPEATS times, with
    # an untimed graph of 2 x `steps` launches between two takes, and the median is reported.
    # Measured alternatives for 20 launches, on boxes where 3000 steps give 7.6 to 7.7 us: the graph
    # of 20 alone after a synchronisation pays its start (8.3 us per launch); launched directly, one
    # host call per kernel, the host is the limit (8.25); event nodes inside one graph cost about
    # 5 us themselves (7.9 to 8.2); the difference of two graph replays (64 + 20 launches against
    # 64), each after a synchronisation, read 6.6 us on one box and 7.5 to 7.75 on another, because
    # the launches at the end of a replay run at clocks the card does not sustain.  This method:
    # 7.82 to 7.88 where 3000 steps give 7.71.
    graph_len = min(steps, graph_rotations * n_buffers)

    def capture(count, first=0):
        stream.begin_capture()
        for i in range(count):
            launch(first + i)
        g = stream.end_capture()
        g.launch(stream)  # untimed: the first replay uploads the graph
        stream.synchronize()
        return g

    def timed(graphs):
        e0.record(stream)
        for g in graphs:
            g.launch(stream)
        e1.record(stream)
        stream.synchronize()
        return e0.elapsed_ms(e1)

    short_run = steps < 64
    e0, e1 = hiprt.Event(), hiprt.Event()
    if short_run:
        prime, timed_graph, filler = capture(256), capture(steps), capture(2 * steps)
        graphs = [prime, timed_graph, filler]
        marks = [hiprt.Event() for _ in range(2 * SHORT_RUN_REPEATS)]
        hiprt.device_synchronize()
        t0 = time.perf_counter()
        for _ in range(SHORT_RUN_PRIMING):
            prime.launch(stream)
        for r in range(SHORT_RUN_REPEATS):
            marks[2 * r].record(stream)
            timed_graph.launch(stream)
            marks[2 * r + 1].record(stream)
            filler.launch(stream)
        stream.synchronize()
        hiprt.device_synchronize()
        wall_launches = SHORT_RUN_PRIMING * 256 + SHORT_RUN_REPEATS * 3 * steps
        event_ms = float(np.median([marks[2 * r].elapsed_ms(marks[2 * r + 1]) for r in range(SHORT_RUN_REPEATS)]))
    else:
        graphs = [capture(graph_len)] * (steps // graph_len)
        if steps % graph_len:
            graphs.append(capture(steps % graph_len))
        hiprt.device_synchronize()
        t0 = time.perf_counter()
        event_ms = timed(graphs)
        hiprt.device_synchronize()
        wall_launches = steps
    wall_ms = (time.perf_counter() - t0) * 1e3
    for g in set(graphs):
        g.destroy()
    result = y.numpy()
    assert np.all(np.isfinite(result))
    for w in weights:
        w.free()
    stream.destroy()
    bench_gemv.last_mode = (f"graphs of {graph_len} launches replayed" if not short_run else
                            f"a graph of {steps} launches between two events in a busy queue ({SHORT_RUN_PRIMING} replays of "
                            f"a graph of 256 launches go first, nothing synchronises in between), median of "
                            f"{SHORT_RUN_REPEATS} such regions (the wall figure is over all launches of the run)")
    return event_ms / steps, wall_ms / wall_launches


def traffic_probe(ln, launches=8, n_elems=16 * 1024 * 1024):
    """A streaming kernel of known HBM traffic for calibrating the profiler's FETCH_SIZE /
    WRITE_SIZE counters: element-wise negation of 64 MiB of f32 (reads 64 MiB, writes 64 MiB
    per launch, far beyond the 4 MiB-per-XCD L2).  Only run under `--traffic-probe`."""
    from litenn_amd.formats import DT_F32
    src = ln.Tensor.from_numpy(np.ones(n_elems, np.float32))
    dst = ln.Tensor((n_elems,))
    for _ in range(launches):
        ln.DeviceTraits.DoUnaryOp(ln.HIP(0), 0, dst.ptr, DT_F32, (n_elems,), src.ptr)  # 0 = Negate
    assert float(dst.numpy()[12345]) == -1.0
    src.free()
    dst.free()
    log(f"[bench] traffic probe: {launches} launches of unary_kernel<float>, {4 * n_elems} B read + "
        f"{4 * n_elems} B written each")


SHORT_RUN_PRIMING = 8  # replays of a graph of 256 launches that precede the timed graph of a short run
SHORT_RUN_REPEATS = 15


FP16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 matrix rate


def bench_gemm(ln, hiprt, fmt, n, k, m, iters=40, n_buffers=8, seed=7):
    """Prefill matmul Y[m,n] = X[m,k] . deq(W)^T on the matrix cores, rotating weight buffers;
    returns the HIP-event time per call in ms (the fp16 pre-pass of X included)."""
    from litenn_amd import synth
    from litenn_amd._lib import Exec, check, load
    import ctypes as C

    lib = load()
    wq_host = synth.quant_weights(fmt, n, k, seed)
    weights = [ln.Tensor.from_numpy(np.roll(wq_host, b, axis=0).reshape(-1)) for b in range(n_buffers)]
    x = ln.Tensor.from_numpy(synth.activations(m, k, seed + 1))
    y = ln.Tensor((m, n))
    # the fp16 copy of the activations, plus room for three more products: lets the library walk K
    # in parts at once where a single walk would leave the card short of work
    ws_bytes = (lib.litenn_hip_mul_mat_q_workspace_bytes(m, k) + 15) // 16 * 16 + 3 * 4 * m * n
    ws = ln.Tensor((ws_bytes // 4,))
    stream = hiprt.Stream()
    opts = Exec(stream.handle, 0)

    def launch(i):
        check(lib.litenn_hip_mul_mat_q_ws(0, fmt, weights[i % n_buffers].ptr, n, k, x.ptr, 0, m, y.ptr, None, 0,
                                          ws.ptr, ws_bytes, C.byref(opts)))

    for i in range(n_buffers):
        launch(i)
    stream.synchronize()
    e0, e1 = hiprt.Event(), hiprt.Event()
    e0.record(stream)
    for i in range(iters):
        launch(i)
    e1.record(stream)
    stream.synchronize()
    ms = e0.elapsed_ms(e1) / iters
    assert np.all(np.isfinite(y.numpy()))
    for w in weights:
        w.free()
    for t in (x, y, ws):
        t.free()
    stream.destroy()
    return ms


def bench_prefill_gemm(ln, hiprt, only=None):
    """only: "FORMAT:M" restricts the run to one case (profiling)."""
    from litenn_amd.formats import Q4_K, Q6_K, row_bytes
    out = []
    for name, fmt, n, k in (("Q4_K", Q4_K, 14336, 4096), ("Q6_K", Q6_K, 4096, 4096)):
        for m in (16, 64, 512):
            if only and only != f"{name}:{m}":
                continue
            ms = bench_gemm(ln, hiprt, fmt, n, k, m)
            flops = 2.0 * m * n * k
            bytes_ = n * row_bytes(fmt, k) + 4 * m * k + 4 * m * n
            out.append({"format": name, "m": m, "n": n, "k": k, "us": round(ms * 1e3, 2),
                        "tflops": round(flops / (ms * 1e-3) / 1e12, 1),
                        "frac_of_fp16_mfma_peak": round(flops / (ms * 1e-3) / 1e12 / FP16_MFMA_PEAK_TFLOPS, 4),
                        "gbps": round(bytes_ / (ms * 1e-3) / 1e9, 1), "launch": last_gemm_launch()})
            log(f"[bench] GEMM {name} M={m} N={n} K={k}: {ms * 1e3:.1f} us, {out[-1]['tflops']} TFLOP/s, "
                f"{out[-1]['gbps']} GB/s; {out[-1]['launch']}")
    return out


def microbench(ln, hiprt, fmt, n, k, n_buffers=16, replays=8):
    """What the headline GEMV's time is made of, measured on the same card with the same rotation of
    weight buffers and the same graph replay (lib/liblitenn_hip_trace.so: the library with timeline
    stamps compiled into the streaming kernel, plus csrc/microbench.hip):
      * a kernel that does nothing, per graph node;
      * a kernel that only reads the same 33 MB per launch (best of several geometries);
      * the streaming kernel's own timeline: per wavefront, on the card's shared 100 MHz clock, when
        it started, had its activations in registers, saw each of its rows land and finished."""
    import ctypes as C
    from litenn_amd import synth
    from litenn_amd import build as hip_build
    from litenn_amd._lib import Exec
    from litenn_amd.formats import row_bytes
    tl = C.CDLL(hip_build.TRACE_LIB_PATH)
    tl.litenn_hip_last_error.restype = C.c_char_p
    vp, sz = C.c_void_p, C.c_size_t
    tl.litenn_hip_mul_mat_q.argtypes = [C.c_int, C.c_int, vp, sz, sz, vp, C.c_int, sz, vp, vp, C.c_uint, C.POINTER(Exec)]
    tl.litenn_hip_mb_empty.argtypes = [C.c_int, C.c_int, sz, vp]
    tl.litenn_hip_mb_read.argtypes = [vp, sz, C.c_int, C.c_int, vp, vp]
    tl.litenn_hip_mb_read_policy.argtypes = [vp, sz, C.c_int, C.c_int, C.c_int, vp, vp]
    tl.litenn_hip_gemv_trace_read.argtypes = [vp, sz]
    tl.litenn_hip_gemv_trace_skip_arithmetic.argtypes = [C.c_int]

    def ok(rc):
        if rc != 0:
            raise RuntimeError(tl.litenn_hip_last_error().decode())

    wq_host = synth.quant_weights(fmt, n, k, 1)
    weights = [ln.Tensor.from_numpy(np.roll(wq_host, b, axis=0).reshape(-1)) for b in range(n_buffers)]
    w_bytes = n * row_bytes(fmt, k)
    x = ln.Tensor.from_numpy(synth.activations(1, k, 2))
    y = ln.Tensor((1, n))
    sink = ln.Tensor((4,))
    stream = hiprt.Stream()
    opts = Exec(stream.handle, 0)

    graph_len = 16 * n_buffers

    def per_launch_us(launch):
        """16 rotations captured as one graph, replayed; HIP events on the stream."""
        for i in range(n_buffers):
            launch(i)
        stream.synchronize()
        stream.begin_capture()
        for i in range(graph_len):
            launch(i)
        graph = stream.end_capture()
        graph.launch(stream)
        stream.synchronize()
        e0, e1 = hiprt.Event(), hiprt.Event()
        e0.record(stream)
        for _ in range(replays):
            graph.launch(stream)
        e1.record(stream)
        stream.synchronize()
        us = e0.elapsed_ms(e1) * 1e3 / (replays * graph_len)
        graph.destroy()
        return us

    out = {"rotation": f"{n_buffers} buffers x {w_bytes} B, graph of {graph_len} launches replayed {replays} times"}
    out["empty_kernel_us"] = round(per_launch_us(lambda i: ok(tl.litenn_hip_mb_empty(256, 512, 90 * 1024,
                                                                                      stream.handle))), 3)
    out["empty_kernel_one_workgroup_us"] = round(per_launch_us(lambda i: ok(tl.litenn_hip_mb_empty(1, 64, 0,
                                                                                                    stream.handle))), 3)
    reads = []
    for blocks in (256, 512, 1024, 2048):
        for depth in (2, 4, 8):
            us = per_launch_us(lambda i: ok(tl.litenn_hip_mb_read(weights[i % n_buffers].ptr, w_bytes, blocks, depth,
                                                                  sink.ptr, stream.handle)))
            reads.append({"blocks": blocks, "loads_in_flight_per_lane": depth, "us": round(us, 3),
                          "gbps": round(w_bytes / us / 1e3, 1)})
    best = min(reads, key=lambda r: r["us"])
    out["read_kernel_best"] = best
    out["read_kernel_all"] = reads
    # the same with non-temporal loads (the policy of the GEMV's weight rows)
    reads_nt = []
    for blocks in (256, 512, 1024, 2048):
        for depth in (2, 4, 8):
            us = per_launch_us(lambda i: ok(tl.litenn_hip_mb_read_policy(weights[i % n_buffers].ptr, w_bytes, blocks,
                                                                         depth, 1, sink.ptr, stream.handle)))
            reads_nt.append({"blocks": blocks, "loads_in_flight_per_lane": depth, "us": round(us, 3),
                             "gbps": round(w_bytes / us / 1e3, 1)})
    best_nt = min(reads_nt, key=lambda r: r["us"])
    out["read_kernel_nontemporal_best"] = best_nt
    out["read_kernel_nontemporal_all"] = reads_nt
    log(f"[bench] microbench: empty kernel {out['empty_kernel_us']} us/launch (one workgroup of 64 threads: "
        f"{out['empty_kernel_one_workgroup_us']}); read-only kernel best "
        f"{best['us']} us = {best['gbps']} GB/s ({best['blocks']} workgroups, {best['loads_in_flight_per_lane']} loads/lane); "
        f"with non-temporal loads {best_nt['us']} us = {best_nt['gbps']} GB/s ({best_nt['blocks']} workgroups, "
        f"{best_nt['loads_in_flight_per_lane']} loads/lane)")

    def gemv(i):
        ok(tl.litenn_hip_mul_mat_q(0, fmt, weights[i % n_buffers].ptr, n, k, x.ptr, 0, 1, y.ptr, None, 0, C.byref(opts)))

    out["gemv_with_stamps_us"] = round(per_launch_us(gemv), 3)
    # the same kernel fetching its rows and reading them from LDS without multiplying them
    ok(tl.litenn_hip_gemv_trace_skip_arithmetic(1))
    out["gemv_with_stamps_no_arithmetic_us"] = round(per_launch_us(gemv), 3)
    ok(tl.litenn_hip_gemv_trace_skip_arithmetic(0))
    log(f"[bench] microbench: streaming kernel with stamps {out['gemv_with_stamps_us']} us/launch, its row traffic "
        f"alone (no arithmetic) {out['gemv_with_stamps_no_arithmetic_us']} us/launch")
    # the timeline of one launch in the middle of a replay: stamps are cleared by the read, then one
    # rotation runs and the last launch's stamps (every launch overwrites them) are read back
    slots = 16
    waves = 256 * 8
    buf = (C.c_ulonglong * (waves * slots))()
    ok(tl.litenn_hip_gemv_trace_read(buf, waves * slots))
    acc = []
    for _ in range(8):
        for i in range(n_buffers):
            gemv(i)
        ok(tl.litenn_hip_gemv_trace_read(buf, waves * slots))
        t = np.frombuffer(buf, np.uint64).reshape(waves, slots).astype(np.float64)
        t = np.where(t == 0, np.nan, t)
        acc.append((t - np.nanmin(t[:, 0])) * 0.01)  # 100 MHz ticks -> us after the first wavefront's entry
    t = np.stack(acc)  # [launch, wavefront, slot]
    names = ["entry", "activations written to LDS", "barrier passed", "activations in registers"] + \
            [f"row {r} landed" for r in range(11)] + ["last row consumed"]
    timeline = []
    for slot, name in enumerate(names):
        col = t[:, :, slot]
        if np.all(np.isnan(col)):
            continue
        timeline.append({"point": name, "mean_us": round(float(np.nanmean(col)), 2),
                         "earliest_us": round(float(np.nanmean(np.nanmin(col, axis=1))), 2),
                         "latest_us": round(float(np.nanmean(np.nanmax(col, axis=1))), 2)})
        log(f"[bench] microbench: {name:28s} mean {timeline[-1]['mean_us']:5.2f} us  earliest "
            f"{timeline[-1]['earliest_us']:5.2f}  latest {timeline[-1]['latest_us']:5.2f}")
    out["gemv_timeline"] = timeline
    # wavefronts 0-3 of a workgroup are the first on their SIMD, 4-7 share it with them
    by_wave = np.nanmean(t[:, :, 15].reshape(len(acc), -1, 8), axis=(0, 1))
    out["last_row_consumed_by_wavefront_index_us"] = [round(float(v), 2) for v in by_wave]
    log("[bench] microbench: last row consumed, by wavefront index within the workgroup: "
        + " ".join(f"{v:.2f}" for v in by_wave))
    out["gemv_timeline_note"] = ("us after the launch's first wavefront entered the kernel, averaged over 8 launches x "
                                 "2048 wavefronts; earliest / latest are the per-launch extremes, averaged")
    # The matrix-core GEMM's instruction mix without its memory traffic: cycles per MFMA and SIMD
    tl.litenn_hip_mb_mix.argtypes = [C.c_int] * 4 + [vp, C.c_int, C.c_int, C.c_int, vp]
    cyc = ln.Tensor((2 * 4608,))  # 4608 counters of 8 bytes
    steps, blocks = 2000, 256
    mix = []
    for threads in (256, 512):
        for (mfma, reads, valu) in ((1, 0, 0), (1, 1, 0), (1, 0, 5), (1, 1, 3), (1, 1, 5), (1, 1, 8)):
            ok(tl.litenn_hip_mb_mix(mfma, reads, valu, 1, cyc.ptr, blocks, threads, steps, stream.handle))
            stream.synchronize()
            raw = cyc.numpy().view(np.uint64)[: blocks * 8].reshape(blocks, 8)[:, : threads // 64].astype(np.float64)
            per_simd = threads // 256                      # wavefronts that share a SIMD
            per_mfma = float(raw.max(axis=1).mean()) / (steps * 16 * per_simd)
            mix.append({"wavefronts_per_simd": per_simd, "lds_reads_per_2_mfma": reads, "valu_per_2_mfma": valu,
                        "cycles_per_mfma_per_simd": round(per_mfma, 2)})
            log(f"[bench] microbench: mix of 2 MFMA + {reads} ds_read_b128 + {valu} VALU, {per_simd} wavefront(s) per SIMD, "
                f"barrier every 64 MFMAs: {per_mfma:.1f} cycles per MFMA and SIMD")
    out["mfma_mix"] = mix
    out["mfma_mix_note"] = ("v_mfma_f32_16x16x32_f16 from registers, fragment reads from LDS, independent f32 multiply-adds; "
                            "256 workgroups, shader-clock cycles of the slowest wavefront of a workgroup")
    cyc.free()
    out["xcd_exchange"] = xcd_exchange(ln, hiprt, tl, ok, stream)
    # the decoder-block kernel's timeline needs the timeline build as THE library: a child process
    import subprocess
    child = subprocess.run([sys.executable, os.path.abspath(__file__), "--block-timeline"], capture_output=True, text=True,
                           timeout=300)
    if child.returncode == 0 and child.stdout.strip():
        out["block_timeline"] = json.loads(child.stdout.strip().splitlines()[-1])
        for pt in out["block_timeline"]["timeline"]:
            log(f"[bench] microbench: decoder-block kernel, {pt['point']:40s} mean {pt['mean_us']:6.2f} us  earliest "
                f"{pt['earliest_us']:6.2f}  latest {pt['latest_us']:6.2f}")
    else:
        log("[bench] microbench: the decoder-block timeline did not run: " + child.stderr.strip()[-300:])
    for w in weights:
        w.free()
    for tns in (x, y, sink):
        tns.free()
    stream.destroy()
    return out


def xcd_exchange(ln, hiprt, tl, ok, stream, phases=2000, blocks=256):
    """What a phase boundary inside one launch costs when only the workgroups of one XCD (32 CUs that
    share an L2) have to meet: 256 workgroups, one per CU, each publishing one value per phase and
    collecting the 32 values of its own XCD (csrc/microbench.hip, mb_xcd_exchange_kernel)."""
    import ctypes as C
    vp = C.c_void_p
    tl.litenn_hip_mb_xcd_exchange.argtypes = [C.c_int] * 5 + [vp] * 5
    mem, err = ln.Tensor((2048 + 512 * phases,)), ln.Tensor((4,))
    result, stamps = ln.Tensor((2 * blocks,)), ln.Tensor((2 * phases,))
    want = 1
    for _ in range(phases):
        want = (32 * want + 1) & 0xFFFFFFFF
    out = []
    for mode, name in ((0, "counter in the L2, values loaded past the L1"),
                       (1, "values carry their phase, polled past the L1"),
                       (2, "values carry their phase, device-scope loads and stores"),
                       (3, "a flag per workgroup polled by atomics in the L2, values by ordinary stores and loads"),
                       (4, "a flag per workgroup polled by device-scope loads, values by ordinary stores and loads")):
        best = None
        for rep in range(3):
            e0, e1 = hiprt.Event(), hiprt.Event()
            e0.record(stream)
            ok(tl.litenn_hip_mb_xcd_exchange(mode, blocks, phases, 4000, 32, mem.ptr, err.ptr, result.ptr, stamps.ptr,
                                              stream.handle))
            e1.record(stream)
            stream.synchronize()
            us = e0.elapsed_ms(e1) * 1e3
            best = us if best is None else min(best, us)
        flag = int(err.numpy().view(np.int32)[0])
        res = result.numpy().view(np.uint32).reshape(blocks, 2)
        per_xcd = np.bincount(res[:, 1] // 64, minlength=8).tolist()
        ticks = stamps.numpy().view(np.uint64)[:phases].astype(np.float64)
        per_phase = float(np.median(np.diff(ticks))) * 0.01
        entry = {"mode": name, "phases": phases, "us_per_phase": round(best / phases, 3),
                 "us_per_phase_median_by_clock": round(per_phase, 3), "waits_ran_out": flag,
                 "workgroups_per_xcd": per_xcd, "values_correct": bool(flag == 0 and np.all(res[:, 0] == want))}
        out.append(entry)
        log(f"[bench] microbench: exchange within an XCD, {name}: {entry['us_per_phase']} us per phase "
            f"(median by the card's clock {entry['us_per_phase_median_by_clock']}), waits that ran out: {flag}, "
            f"workgroups per XCD {per_xcd}, values correct: {entry['values_correct']}")
    for t in (mem, err, result, stamps):
        t.free()
    return out


def block_timeline(past=200, steps=6):
    """The decoder-block kernel's own timeline (csrc/attn_block.inc) from the timeline build of the library:
    a four-block model of the 7B shape's attention half (4096 wide, 32 heads of 128, Q4_0, small
    feed-forward part and vocabulary), `past` cached rows, single-token steps launched kernel by
    kernel; the last block's launch of every step leaves its stamps.  Runs in a process of its own
    (`python bench.py --block-timeline`): the library this process loads is the timeline build."""
    import ctypes as C
    os.environ["LITENN_HIP_GRAPH"] = "0"
    from litenn_amd import _lib, build as hip_build
    _lib.LIB_PATH = hip_build.TRACE_LIB_PATH
    import litenn_amd as ln
    from litenn_amd import synth
    from litenn_amd.formats import DT_F16, Q4_0
    cfg = synth.tiny_llama(Q4_0, block_count=4, d_model=4096, heads=32, kv_heads=32, ff=256, vocab=256,
                           context_length=past + steps + 8)
    model = ln.LLaMA.from_config(cfg, kv_dtype=DT_F16)
    for item in synth.llama_tensors(cfg, 3):
        model.set_tensor(*item)
    toks = synth.prompt_tokens(cfg, past + steps + 2, 1)
    model.eval(toks[:past], all_logits=False, precise=False)
    lib = _lib.load()
    lib.litenn_hip_block_trace_read.argtypes = [C.c_void_p, C.c_size_t]
    waves, slots = 2048, 8
    buf = (C.c_ulonglong * (waves * slots))()
    acc = []
    for t in toks[past:past + steps + 2]:
        model.eval([t], all_logits=False)
        if lib.litenn_hip_block_trace_read(buf, waves * slots) != 0:
            raise RuntimeError(lib.litenn_hip_last_error().decode())
        a = np.frombuffer(buf, np.uint64).reshape(waves, slots).astype(np.float64)
        acc.append((a - a[:, 0].min()) * 0.01)  # 100 MHz ticks -> us after the launch's first wavefront entered
    form = model.block_form
    model.close()
    a = np.stack(acc[2:])
    names = ["entry", "first phase's rows stored", "first meeting passed", "second phase's triple stored",
             "second meeting passed", "third phase's activations in registers", "end"]
    points = []
    for s_, name in enumerate(names):
        col = a[:, :, s_]
        points.append({"point": name, "mean_us": round(float(col.mean()), 2),
                       "earliest_us": round(float(col.min(axis=1).mean()), 2),
                       "latest_us": round(float(col.max(axis=1).mean()), 2)})
    return {"block_form": form, "cached_rows": past, "steps": steps, "timeline": points,
            "note": "us after the launch's first wavefront entered the kernel, over all 2048 wavefronts of the last "
                    "block's launch; earliest / latest are per-launch extremes, averaged over the steps"}


def bench_cpu_baseline(fmt, n, k, budget_s=8.0):
    """The reference CPU path for the same GEMV, restated by the CPU checker, timed on this host:
      * one-off: block dequantisation to f32 [n, k] and the transpose to [k, n] that the lowering does
        once per graph (tools/gguf/LLaMABuilder.cpp:144-150, 225-230);
      * per call, one thread: the i-k-j MatMul of src/LiteNN/Device.h:645-658 on that f32 matrix;
      * per call, one thread, with the copy of the weight variable the Interpreter makes at every
        VariableRefNode first (src/LiteNN/Runtime/Interpreter.h:325-329);
      * not the reference: the checker's OpenMP form (rows dequantised on the fly, all cores)."""
    from litenn_amd import synth
    from oracle import oracle as orc
    orc.set_threads(1)
    wq = synth.quant_weights(fmt, n, k, 1)
    x = synth.activations(1, k, 2)
    t0 = time.perf_counter()
    w_kn = orc.transpose(orc.dequantize(fmt, wq, n, k))
    dequant_s = time.perf_counter() - t0
    orc.matmul_ikj(x, w_kn)  # warm

    def timed(fn, budget):
        calls, t0 = 0, time.perf_counter()
        while True:
            fn()
            calls += 1
            dt = time.perf_counter() - t0
            if dt > budget or calls >= 2000:
                return dt / calls, calls

    s_per_call, calls = timed(lambda: orc.matmul_ikj(x, w_kn), budget_s)
    s_with_copy, calls_copy = timed(lambda: orc.matmul_ikj(x, w_kn.copy()), budget_s / 2)
    cores = os.cpu_count() or 1
    orc.set_threads(cores)
    orc.mul_mat_q(fmt, wq, n, k, x, rowwise=True)
    s_omp, calls_omp = timed(lambda: orc.mul_mat_q(fmt, wq, n, k, x, rowwise=True), budget_s / 2)
    return {"s_per_call": s_per_call, "calls": calls, "s_with_copy": s_with_copy, "calls_copy": calls_copy,
            "dequant_s": dequant_s, "s_omp": s_omp, "calls_omp": calls_omp, "omp_threads": cores}


ORACLE_TENSOR_IDS = {"token_embd": 0, "output": 1, "attn_q": 2, "attn_k": 3, "attn_v": 4, "attn_output": 5,
                     "ffn_gate": 6, "ffn_up": 7, "ffn_down": 8, "output_norm": 9, "attn_norm": 10, "ffn_norm": 11}


FIXTURE_7B = os.path.join(ROOT, "tests", "golden", "llama7b_q4_0_tokens.json")


def cpu_decode_rate(cfg, tensors, prompt, steps, threads):
    """Tokens per second of the CPU checker's decoder on the same model: `steps` single-token
    evaluations behind a one-token prompt, on `threads` threads.  One thread is the reference's
    case (its Interpreter and DeviceTraits<CPU> are single-threaded,
    src/LiteNN/Runtime/Interpreter.h:89-104, src/LiteNN/Device.h:645-658); the checker dequantises
    each row on the fly where the reference multiplies f32 weights dequantised at lowering, the same
    f32 sequence per output."""
    from oracle import oracle as orc
    orc.set_threads(threads)
    m = orc.LLaMA(cfg.block_count, cfg.embedding_length, cfg.head_count, cfg.head_count_kv, cfg.feed_forward_length,
                  cfg.vocab, cfg.context_length, rms_eps=cfg.rms_eps, rope_base=cfg.rope_freq_base,
                  rope_freq_scale=cfg.rope_freq_scale, rope_dims=cfg.rope_dimension_count, kv_f16=True)
    for kind, layer, fmt, payload, n, k in tensors:
        m.set_tensor(ORACLE_TENSOR_IDS[kind], layer, fmt, payload, n, k)
    logits = m.eval([int(prompt[0])], all_logits=False)
    t0 = time.perf_counter()
    for _ in range(steps):
        logits = m.eval([int(np.argmax(logits))], all_logits=False)
    dt = time.perf_counter() - t0
    return steps / dt


def fixture_7b(n_prompt, n_new):
    """The committed token fixture of the 7B-shape run (written from the CPU checker by
    tests/golden/make_llama7b_tokens.py; data, not code), when it covers these lengths."""
    try:
        with open(FIXTURE_7B) as f:
            fx = json.load(f)
    except OSError:
        return None
    if not fx.get("complete") or fx["prompt_length"] != n_prompt or fx["new_tokens"] < n_new:
        return None
    return fx


def bench_decode(ln, n_prompt=128, n_new=256, seed=4, model_name="7b", cpu_steps=0):
    from litenn_amd import synth
    from litenn_amd.formats import DT_F16
    fx = None
    if model_name == "8b":
        cfg = synth.llama_8b_gqa_mixed(context_length=max(4096, n_prompt + n_new))
    else:
        cfg = synth.llama_7b_q4_0(context_length=n_prompt + n_new)
        fx = fixture_7b(n_prompt, n_new)
    prompt_seed = seed
    if fx is not None and fx["model"] == cfg.name and fx["context_length"] == cfg.context_length:
        # the model and the prompt of the fixture, so that the timed run's tokens can be held to it
        seed, prompt_seed = fx["seed"], fx["prompt_seed"]
    else:
        fx = None
    t0 = time.perf_counter()
    model = ln.LLaMA.from_config(cfg, kv_dtype=DT_F16)
    tensors = []
    for item in synth.llama_tensors(cfg, seed):
        model.set_tensor(*item)
        if cpu_steps:
            tensors.append(item)
    log(f"[bench] {cfg.name} resident after {time.perf_counter() - t0:.1f} s")
    prompt = synth.prompt_tokens(cfg, n_prompt, prompt_seed)
    model.generate(prompt, 8, precise=False)  # warm-up: captures the step graph
    model.reset()
    # prompt pass on the matrix cores (fp16 operands), then the captured single-token step
    tokens, prefill_ms, decode_ms = model.generate(prompt, n_new, precise=False)
    steps = n_new - 1
    weight_bytes = cfg.matmul_weight_bytes_per_token()
    kv_bytes_mean = 2 * cfg.block_count * cfg.head_count_kv * cfg.head_dim * 2 * (n_prompt + n_new / 2)
    tok_s = steps / (decode_ms / 1e3)
    out = {
        "workload": f"{cfg.name}: prompt {n_prompt} + {n_new} greedy tokens, context {cfg.context_length}, "
                    f"fp16 KV cache, f32 activations, model seed {seed}, prompt seed {prompt_seed}",
        "tokens_per_s": round(tok_s, 2),
        "ms_per_token": round(decode_ms / steps, 4),
        "prefill_ms": round(prefill_ms, 3),
        "prefill_tokens_per_s": round(n_prompt / (prefill_ms / 1e3), 1),
        "prompt_pass": "matrix cores, Float16 operands (flags = 0, the C ABI's default)",
        "weight_bytes_per_token": weight_bytes,
        "roofline_tokens_per_s": round(HBM_PEAK_GBPS * 1e9 / (weight_bytes + kv_bytes_mean), 1),
        "frac_of_hbm_roofline": round(tok_s * (weight_bytes + kv_bytes_mean) / (HBM_PEAK_GBPS * 1e9), 4),
        "distinct_tokens": int(len(set(tokens.tolist()))),
        "first_tokens": tokens[:8].tolist(),
    }
    if fx is not None:
        want = np.array(fx["tokens"][:n_new])
        same = tokens == want
        first_off = int(np.argmin(same)) if not same.all() else n_new
        out["tokens_matching_fixture"] = int(same.sum())
        out["fixture"] = {"file": os.path.relpath(FIXTURE_7B, ROOT), "tokens": int(n_new),
                          "matching": int(same.sum()), "matching_prefix": first_off,
                          "source": fx.get("source"),
                          "note": "the timed run's tokens against the CPU checker's; its prompt pass has Float16 "
                                  "operands, the fixture's Float32 ones"}
        if first_off < n_new:
            out["fixture"]["checker_margin_at_first_difference"] = fx["margins"][first_off]
        # the same generation behind the Float32-operand prompt pass (untimed): the path the reference's
        # arithmetic is restated on
        model.reset()
        exact, _, _ = model.generate(prompt, n_new, precise=True)
        out["fixture"]["matching_with_f32_prompt_pass"] = int((exact == want).sum())
        log(f"[bench] tokens matching the committed fixture: {out['tokens_matching_fixture']} of {n_new} "
            f"(Float32 prompt pass: {out['fixture']['matching_with_f32_prompt_pass']})")
    model.close()
    if cpu_steps:
        cores = os.cpu_count() or 1
        rate_all = cpu_decode_rate(cfg, tensors, prompt, cpu_steps, cores)
        rate_one = cpu_decode_rate(cfg, tensors, prompt, max(1, cpu_steps // 2), 1)
        out["cpu_tokens_per_s"] = round(rate_one, 4)
        out["cpu_baseline"] = {"value": round(rate_one, 4), "unit": "tokens/s", "cores": 1, "kind": "port",
                               "sample": f"{max(1, cpu_steps // 2)} single-token steps of the CPU checker's decoder on "
                                         f"the same model on one thread (the reference's interpreter is "
                                         f"single-threaded), rows dequantised on the fly",
                               "all_cores": {"value": round(rate_all, 3), "unit": "tokens/s", "cores": cores,
                                             "kind": "port-omp (not the reference)",
                                             "sample": f"{cpu_steps} steps of the same decoder on {cores} threads"}}
    return out


def bench_gemv_configs(ln, hiprt, steps=1600, warmup=64):
    """The other single-row configurations: Q8_0 4096 x 4096 and the Q4_0 / Q4_K FFN shapes, each
    with its own roofline object (rotating buffers of more than 512 MB in total)."""
    from litenn_amd.formats import Q4_0, Q4_K, Q8_0, row_bytes
    out = []
    traffic = measured_config_traffic()
    for name, fmt, n, k in (("Q8_0", Q8_0, 4096, 4096), ("Q4_0", Q4_0, 11008, 4096), ("Q4_0", Q4_0, 4096, 11008),
                            ("Q4_K", Q4_K, 11008, 4096), ("Q4_K", Q4_K, 4096, 11008)):
        w_bytes = n * row_bytes(fmt, k)
        buffers = max(16, -(-540_000_000 // w_bytes))
        ms, _ = bench_gemv(ln, hiprt, fmt, n, k, steps // buffers * buffers, warmup, buffers)
        algo = w_bytes + 4 * k + 4 * n
        gbps = algo / (ms * 1e-3) / 1e9
        out.append({"format": name, "n": n, "k": k, "batch": 1, "us": round(ms * 1e3, 3), "buffers": buffers,
                    "algorithmic_bytes": algo,
                    "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                 "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": traffic.get((name, n, k))}})
        log(f"[bench] {name} GEMV {n}x{k}: {ms * 1e3:.2f} us/launch, {gbps:.0f} GB/s = "
            f"{100 * gbps / HBM_PEAK_GBPS:.1f}% of HBM peak")
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--buffers", type=int, default=16)
    ap.add_argument("--graph-rotations", type=int, default=16,
                    help="rotations of the weight buffers one replayed graph holds (the profiler slows long graphs "
                         "down a great deal: its runs use 1)")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the other single-row GEMV configurations")
    ap.add_argument("--config-steps", type=int, default=1600, help="launches timed per other GEMV configuration")
    ap.add_argument("--decode-prompt", type=int, default=128, help="prompt length of the decode run")
    ap.add_argument("--decode-new", type=int, default=256, help="tokens generated by the decode run")
    ap.add_argument("--decode-model", choices=["7b", "8b", "both"], default="both",
                    help="7b: 7B-shape Q4_0 at --decode-prompt / --decode-new; 8b: 8B GQA shape, Q4_K + Q6_K, at the "
                         "same lengths; both (default): the 7B shape at those lengths and the 8B shape at prompt 512 "
                         "+ 512 tokens")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-gemm", action="store_true", help="skip the prefill (batched matmul) measurements")
    ap.add_argument("--gemm-case", default=None, help="run only this prefill case, e.g. Q4_K:512")
    ap.add_argument("--microbench", action="store_true",
                    help="also measure an empty kernel, a read-only kernel and the GEMV's in-kernel timeline")
    ap.add_argument("--block-timeline", action="store_true",
                    help="print the decoder-block kernel's in-kernel timeline (timeline build of the library) and exit")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also launch a known-size streaming kernel (profiler counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has nothing sharded or exchanged between GPUs; "
              "run with --gpus 1", file=sys.stderr)
        return 2

    if args.block_timeline:
        print(json.dumps(block_timeline()), flush=True)
        return 0

    import litenn_amd as ln
    from litenn_amd import hiprt
    from litenn_amd.formats import Q4_K, row_bytes

    if ln.HIPDeviceCount() == 0:
        print("bench.py needs a HIP device", file=sys.stderr)
        return 1
    log("[bench]", ln.DeviceTraits.Info(ln.HIP(0)))

    if args.traffic_probe:
        traffic_probe(ln)

    n, k = 14336, 4096
    algo_bytes = n * row_bytes(Q4_K, k) + 4 * k + 4 * n
    ms_event, ms_wall = bench_gemv(ln, hiprt, Q4_K, n, k, args.steps, args.warmup, args.buffers,
                                   graph_rotations=max(1, args.graph_rotations))
    gbps = algo_bytes / (ms_event * 1e-3) / 1e9
    launch_mode = bench_gemv.last_mode
    launched = last_gemv_launch()
    log(f"[bench] kernel: {launched}")
    log(f"[bench] Q4_K GEMV {n}x{k}: {ms_event * 1e3:.2f} us/launch (events), {ms_wall * 1e3:.2f} us (wall), "
        f"{gbps:.0f} GB/s = {100 * gbps / HBM_PEAK_GBPS:.1f}% of HBM peak")

    line = {
        "metric": "Q4_K GEMV HBM GB/s (% peak) + decode tokens/s, 7B-shape Q4_0, 1 GPU",
        "value": round(gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_event, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"Q4_K GEMV W[{n}x{k}] . x[{k}], batch 1, {args.buffers} rotating weight buffers "
                        f"({args.buffers * n * row_bytes(Q4_K, k) / 1e6:.0f} MB), one launch per step, "
                        f"{launch_mode}",
            "format": "Q4_K", "n": n, "k": k, "batch": 1, "algorithmic_bytes_per_step": algo_bytes,
            "pct_of_hbm_peak": round(100 * gbps / HBM_PEAK_GBPS, 2),
            "wall_ms_per_step": round(ms_wall, 6),
        },
        "roofline": {
            "bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": measured_traffic_bytes(),
            "traffic_unit": "bytes/launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated)",
            "traffic_source": traffic_source(),
            "algorithmic_bytes": algo_bytes,
            "kernel": launched.split(" grid ")[0],
            "launch": launched,
        },
    }
    if args.microbench:
        line["microbench"] = microbench(ln, hiprt, Q4_K, n, k, args.buffers)
    if not args.no_cpu:
        c = bench_cpu_baseline(Q4_K, n, k)
        line["cpu_baseline"] = {
            "value": round(algo_bytes / c["s_per_call"] / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{c['calls']} calls of the same {n}x{k} GEMV: weights dequantised once to f32 [k,n], then the "
                      f"single-threaded i-k-j MatMul ({c['s_per_call'] * 1e3:.1f} ms/call); host has "
                      f"{os.cpu_count()} logical CPUs",
            "ms_per_step": round(c["s_per_call"] * 1e3, 3),
            "with_weight_copy": {"value": round(algo_bytes / c["s_with_copy"] / 1e9, 4), "unit": "GB/s", "cores": 1,
                                 "ms_per_step": round(c["s_with_copy"] * 1e3, 3),
                                 "sample": f"{c['calls_copy']} calls, each preceded by the copy of the f32 weight "
                                           f"the reference's Interpreter makes per VariableRefNode"},
            "dequantise_once_ms": round(c["dequant_s"] * 1e3, 1),
            "all_cores": {"value": round(algo_bytes / c["s_omp"] / 1e9, 4), "unit": "GB/s", "cores": c["omp_threads"],
                          "kind": "port-omp (not the reference)", "ms_per_step": round(c["s_omp"] * 1e3, 3),
                          "sample": f"{c['calls_omp']} calls of the checker's OpenMP form (rows dequantised on the "
                                    f"fly, same arithmetic per output)"},
        }
        log(f"[bench] CPU baseline: {c['s_per_call'] * 1e3:.1f} ms/call on one thread, "
            f"{c['s_with_copy'] * 1e3:.1f} ms with the weight copy, dequantisation once {c['dequant_s'] * 1e3:.0f} ms, "
            f"{c['s_omp'] * 1e3:.1f} ms/call on {c['omp_threads']} threads (not the reference)")
    if not args.no_configs:
        line["gemv_configs"] = bench_gemv_configs(ln, hiprt, steps=args.config_steps)
    if not args.no_gemm:
        line["prefill_gemm"] = bench_prefill_gemm(ln, hiprt, args.gemm_case)
    if not args.no_decode:
        cpu_steps = 0 if args.no_cpu else 4
        if args.decode_model == "8b":
            line["decode_8b"] = bench_decode(ln, args.decode_prompt, args.decode_new, model_name="8b")
        else:
            line["decode"] = bench_decode(ln, args.decode_prompt, args.decode_new, model_name="7b",
                                          cpu_steps=cpu_steps)
            log(f"[bench] decode: {line['decode']['tokens_per_s']} tok/s"
                + (f" (CPU checker on one thread: {line['decode']['cpu_tokens_per_s']} tok/s, on all cores "
                   f"{line['decode']['cpu_baseline']['all_cores']['value']})" if cpu_steps else ""))
            if args.decode_model == "both":
                line["decode_8b"] = bench_decode(ln, 512, 512, model_name="8b")
        if "decode_8b" in line:
            log(f"[bench] decode 8B shape: {line['decode_8b']['tokens_per_s']} tok/s, prompt pass "
                f"{line['decode_8b']['prefill_ms']} ms")
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
