#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline (BASELINE.json metric, configs[1]): Q4_K decode GEMV, weights 14336 x 4096 (Llama-3-8B FFN
up/gate), one token.  A step = one pass of the path over one batch of synthetic input, inputs
already resident in HBM: device-side Q8_K quantisation of the activation + the GEMV, which the library runs
as ONE launch (every workgroup quantises the token itself).
Steps rotate over enough distinct weight copies to exceed the 256 MiB Infinity Cache, so the
weights of every step come from HBM.

Prints ONE JSON line on stdout (progress goes to stderr):
  value      whole-job GB/s = algorithmic bytes per step * K / wall time of K steps
  roofline   that kernel: algorithmic bytes per launch / mean kernel duration, against the 8 TB/s HBM peak.  Kernel
             times come from HIP events on the library's stream over 200 launches after 20 warm-ups, whatever --steps
             says: mean over all of them, median / p10 / p90 over batches of 10.  `read_ceiling` is what a kernel that
             only reads the same bytes reaches in the same run (context; the peak stays 8 TB/s).
  roofline_gemm  the metric's second half: the Q4_K prefill GEMM (512 tokens) against the 5 POP/s int8 peak, with what a
             kernel of int8 matrix instructions alone reaches in the same run beside it
  cpu_baseline  the CPU restatement of rnb-cpu's x86 path (oracle/, AVX2+FMA, row-chunk threads) timed on
             the host cores on the same workload; cpu_baseline_gemm and cpu_baseline_moe for the GEMM and MoE configs
  secondary  the other BASELINE configs (same protocol; `step` = everything one call enqueues)
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBPS = 8000.0
INT8_PEAK_TOPS = 5000.0  # dense int8 MFMA, POP/s -> TOP/s
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
BLOCK_BYTES = {Q8_0: 34, Q4_K: 144, Q5_K: 176, Q6_K: 210}
BLOCK_ELEMS = {Q8_0: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256}
MALL_BYTES = 256 << 20


def log(msg: str) -> None:
    print(msg, file=sys.stderr, flush=True)


# ---- synthetic weights: fp32 N(0, 0.02) fitted to valid GGUF blocks with numpy -------------------
# (block layouts are the real ones; the fit is a plain vectorised min/max fit -- the kernels' speed
# does not depend on the values)

def _f16_bytes(a: np.ndarray) -> np.ndarray:
    return a.astype(np.float16).view(np.uint8).reshape(*a.shape, 2)


def synth_q8_0(rng, rows, cols):
    x = rng.standard_normal((rows, cols // 32, 32), dtype=np.float32) * np.float32(0.02)
    d = (np.abs(x).max(axis=2) / 127.0).astype(np.float16)
    df = np.maximum(d.astype(np.float32), 1e-12)
    q = np.clip(np.rint(x / df[..., None]), -127, 127).astype(np.int8)
    out = np.empty((rows, cols // 32, 34), np.uint8)
    out[..., 0:2] = d.view(np.uint8).reshape(rows, cols // 32, 2)
    out[..., 2:] = q.view(np.uint8)
    return out.reshape(-1)


def _synth_kquant_min(rng, rows, cols, qmax):
    """Shared fit of the Q4_K / Q5_K synthetic generators: header bytes (d, dmin, 12 packed 6-bit scales and mins) and
    the per-element codes 0..qmax as [rows][nb][4 groups][2 halves][32]."""
    nb = cols // 256
    x = rng.standard_normal((rows, nb, 8, 32), dtype=np.float32) * np.float32(0.02)
    lo = np.minimum(x.min(axis=3), 0.0)
    hi = x.max(axis=3)
    scale = (hi - lo) / float(qmax)
    mins = -lo
    d = (scale.max(axis=2) / 63.0).astype(np.float16)
    dmin = (mins.max(axis=2) / 63.0).astype(np.float16)
    df = np.maximum(d.astype(np.float32), 1e-12)[..., None]
    dmf = np.maximum(dmin.astype(np.float32), 1e-12)[..., None]
    sc = np.clip(np.rint(scale / df), 0, 63).astype(np.uint8)
    mn = np.clip(np.rint(mins / dmf), 0, 63).astype(np.uint8)
    step = np.maximum(df * sc, 1e-12)[..., None]
    q = np.clip(np.rint((x + (dmf * mn)[..., None]) / step), 0, qmax).astype(np.uint8)
    hdr = np.empty((rows, nb, 16), np.uint8)
    hdr[..., 0:2] = d.view(np.uint8).reshape(rows, nb, 2)
    hdr[..., 2:4] = dmin.view(np.uint8).reshape(rows, nb, 2)
    hdr[..., 4:8] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    hdr[..., 8:12] = (mn[..., 0:4] & 63) | ((mn[..., 4:8] >> 4) << 6)
    hdr[..., 12:16] = (sc[..., 4:8] & 15) | ((mn[..., 4:8] & 15) << 4)
    return hdr, q.reshape(rows, nb, 4, 2, 32)


def synth_q4_k(rng, rows, cols):
    nb = cols // 256
    hdr, qg = _synth_kquant_min(rng, rows, cols, 15)
    out = np.empty((rows, nb, 144), np.uint8)
    out[..., 0:16] = hdr
    out[..., 16:] = (qg[:, :, :, 0, :] | (qg[:, :, :, 1, :] << 4)).reshape(rows, nb, 128)
    return out.reshape(-1)


def synth_q5_k(rng, rows, cols):
    nb = cols // 256
    hdr, qg = _synth_kquant_min(rng, rows, cols, 31)
    out = np.empty((rows, nb, 176), np.uint8)
    out[..., 0:16] = hdr
    qh = np.zeros((rows, nb, 32), np.uint8)
    for g in range(4):
        for h in range(2):
            qh |= (qg[:, :, g, h, :] >> 4) << (2 * g + h)
    out[..., 16:48] = qh
    out[..., 48:] = ((qg[:, :, :, 0, :] & 15) | ((qg[:, :, :, 1, :] & 15) << 4)).reshape(rows, nb, 128)
    return out.reshape(-1)


def synth_q6_k(rng, rows, cols):
    nb = cols // 256
    x = rng.standard_normal((rows, nb, 16, 16), dtype=np.float32) * np.float32(0.02)
    scale = np.abs(x).max(axis=3) / 31.0
    d = (scale.max(axis=2) / 127.0).astype(np.float16)
    df = np.maximum(d.astype(np.float32), 1e-12)[..., None]
    sc = np.clip(np.rint(scale / df), 1, 127).astype(np.int8)
    q = (np.clip(np.rint(x / (df * sc)[..., None]), -32, 31) + 32).astype(np.uint8)
    q = q.reshape(rows, nb, 2, 4, 32)  # half, quarter, l
    out = np.empty((rows, nb, 210), np.uint8)
    ql = np.empty((rows, nb, 2, 64), np.uint8)
    ql[..., 0:32] = (q[:, :, :, 0] & 15) | ((q[:, :, :, 2] & 15) << 4)
    ql[..., 32:64] = (q[:, :, :, 1] & 15) | ((q[:, :, :, 3] & 15) << 4)
    qh = (q[:, :, :, 0] >> 4) | ((q[:, :, :, 1] >> 4) << 2) | ((q[:, :, :, 2] >> 4) << 4) | ((q[:, :, :, 3] >> 4) << 6)
    out[..., 0:128] = ql.reshape(rows, nb, 128)
    out[..., 128:192] = qh.reshape(rows, nb, 64)
    out[..., 192:208] = sc.view(np.uint8)
    out[..., 208:210] = d.view(np.uint8).reshape(rows, nb, 2)
    return out.reshape(-1)


SYNTH = {Q8_0: synth_q8_0, Q4_K: synth_q4_k, Q5_K: synth_q5_k, Q6_K: synth_q6_k}


def synth_weights(quant, rows, cols, seed, distinct_rows=16384):
    """rows x cols packed weights; beyond `distinct_rows` the generated rows repeat (addresses differ, so
    cache behaviour is that of fully distinct data)."""
    rng = np.random.default_rng(seed)
    gen = min(rows, distinct_rows)
    parts = [SYNTH[quant](rng, min(4096, gen - r0), cols) for r0 in range(0, gen, 4096)]
    base = np.concatenate(parts)
    if gen == rows:
        return base
    reps = -(-rows // gen)
    rb = cols // BLOCK_ELEMS[quant] * BLOCK_BYTES[quant]
    return np.tile(base, reps)[:rows * rb].copy()


# ---- HIP events on the library stream (ctypes on the runtime the library already loaded) ----------

class Hip:
    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.rt.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipEventSynchronize.argtypes = [C.c_void_p]
        self.rt.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.rt.hipEventDestroy.argtypes = [C.c_void_p]
        self.rt.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        self.rt.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        self.rt.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        self.rt.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipGraphExecDestroy.argtypes = [C.c_void_p]
        self.rt.hipGraphDestroy.argtypes = [C.c_void_p]
        self.rt.hipMemcpyAsync.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]

    def check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed with hipError {rc}")

    def event(self):
        ev = C.c_void_p()
        self.check(self.rt.hipEventCreate(C.byref(ev)), "hipEventCreate")
        return ev

    def record(self, ev, stream):
        self.check(self.rt.hipEventRecord(ev, stream), "hipEventRecord")

    def elapsed_ms(self, a, b):
        self.check(self.rt.hipEventSynchronize(b), "hipEventSynchronize")
        ms = C.c_float()
        self.check(self.rt.hipEventElapsedTime(C.byref(ms), a, b), "hipEventElapsedTime")
        return float(ms.value)


KERNEL_LAUNCHES, KERNEL_WARMUPS, KERNEL_BATCH = 200, 20, 10


def kernel_stats(hip, stream, launch, launches=KERNEL_LAUNCHES, warmups=KERNEL_WARMUPS, batch=KERNEL_BATCH):
    """Duration of `launch(i)` in ms from HIP events recorded on the stream the kernels run on: `warmups` untimed
    launches, then `launches` back-to-back ones with an event after every `batch` of them (same-stream launches
    serialise, so a batch's elapsed time / batch is the kernel duration plus the inter-launch gap).  mean = first to
    last event over all launches; median, p10 and p90 are taken over the batches."""
    for i in range(warmups):
        launch(i)
    n_batches = max(1, launches // batch)
    events = [hip.event() for _ in range(n_batches + 1)]
    hip.record(events[0], stream)
    k = 0
    for b in range(n_batches):
        for _ in range(batch):
            launch(k)
            k += 1
        hip.record(events[b + 1], stream)
    total = hip.elapsed_ms(events[0], events[-1])
    per = np.array([hip.elapsed_ms(events[b], events[b + 1]) / batch for b in range(n_batches)])
    for ev in events:
        hip.rt.hipEventDestroy(ev)
    return {"mean": total / (n_batches * batch), "median": float(np.median(per)), "p10": float(np.percentile(per, 10)),
            "p90": float(np.percentile(per, 90)), "launches": n_batches * batch, "warmups": warmups, "batch": batch}


def kernel_time_ms(hip, stream, launch, n):
    """Mean duration of `launch(i)` over n back-to-back launches (one event before, one after)."""
    e0, e1 = hip.event(), hip.event()
    hip.record(e0, stream)
    for i in range(n):
        launch(i)
    hip.record(e1, stream)
    ms = hip.elapsed_ms(e0, e1)
    hip.rt.hipEventDestroy(e0)
    hip.rt.hipEventDestroy(e1)
    return ms / n


def read_ceiling(hip, rnb, stream, nbytes):
    """What a read-only kernel reaches on `nbytes` in this run (plain and non-temporal 16-byte loads), rotating over
    enough buffers to miss the 256 MiB Infinity Cache: context for the HBM-bound rows, not a peak."""
    n = copies_for(nbytes)
    bufs = [rnb.DeviceBuffer(nbytes) for _ in range(n)]
    out = {"bytes": nbytes, "copies": n}
    for label, nt in (("plain", False), ("non_temporal", True)):
        st = kernel_stats(hip, stream, lambda i: rnb.calib_read(bufs[i % n], nbytes, nt))
        out[label] = {"ms_median": st["median"], "ms_p10": st["p10"], "ms_p90": st["p90"], "GB/s": nbytes / st["median"] / 1e6}
    for b in bufs:
        b.free()
    out["GB/s"] = max(out["plain"]["GB/s"], out["non_temporal"]["GB/s"])
    out["frac_of_peak"] = out["GB/s"] / HBM_PEAK_GBPS
    return out


def mfma_ceiling(hip, rnb, stream):
    """What a kernel of int8 matrix instructions alone (registers only, 2 waves per SIMD on every compute unit) reaches in
    this run: the part's clock under matrix load decides it.  Context for the GEMM row, not a peak."""
    ops = [0]

    def launch(_i):
        ops[0] = rnb.calib_mfma_i8(2000, 256)

    st = kernel_stats(hip, stream, launch, launches=40, warmups=5, batch=5)
    return {"ops_per_launch": ops[0], "ms_median": st["median"], "TOP/s": ops[0] / st["median"] / 1e9,
            "frac_of_peak": ops[0] / st["median"] / 1e9 / INT8_PEAK_TOPS}


def calibration_copy(hip, rnb, stream, nbytes=64 << 20, reps=5):
    """A plain device-to-device copy of known size (the runtime's copy kernel): the reference point that the
    FETCH_SIZE / WRITE_SIZE counters of a `rocprofv3 --pmc` run are scaled by."""
    src, dst = rnb.DeviceBuffer(nbytes), rnb.DeviceBuffer(nbytes)
    for _ in range(reps):
        hip.check(hip.rt.hipMemcpyAsync(dst.ptr, src.ptr, nbytes, 3, stream), "hipMemcpyAsync")  # 3 = device to device
    rnb.sync()
    src.free()
    dst.free()
    log(f"calibration copy: {reps} x {nbytes} bytes device-to-device")


def copy_context(hip, rnb, stream, nbytes):
    """Context for the roofline line: what the runtime's own device-to-device copy reaches on buffers of the size of
    one launch's weights (it reads nbytes and writes nbytes), rotating over enough buffer pairs to miss the 256 MiB
    Infinity Cache.  Reported as total traffic (2 * nbytes per copy) over time; informative only."""
    pairs = max(2, -(-2 * MALL_BYTES // (2 * nbytes)))
    bufs = [(rnb.DeviceBuffer(nbytes), rnb.DeviceBuffer(nbytes)) for _ in range(pairs)]

    def one(i):
        src, dst = bufs[i % pairs]
        hip.check(hip.rt.hipMemcpyAsync(dst.ptr, src.ptr, nbytes, 3, stream), "hipMemcpyAsync")

    for i in range(pairs):
        one(i)
    ms = kernel_time_ms(hip, stream, one, 200)
    for a, b in bufs:
        a.free()
        b.free()
    return {"bytes_copied": nbytes, "ms": ms, "read_plus_write_GB/s": 2 * nbytes / ms / 1e6}


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel`, from the committed counter summary (two rocprofv3 --pmc runs, FETCH_SIZE and
    WRITE_SIZE, each scaled by the same counter's reading for the calibration copy); None when absent."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "gemv_q4k_cfg2_hbm_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(kernel, {}).get("traffic_bytes_per_launch")
    except (OSError, ValueError):
        return None


def wall_steps(rnb, step, n):
    rnb.sync()
    t0 = time.perf_counter()
    for i in range(n):
        step(i)
    rnb.sync()
    return (time.perf_counter() - t0) * 1e3


def graph_steps(hip, rnb, stream, step, per_graph, n_graphs):
    """Capture `per_graph` steps into one HIP graph and replay it `n_graphs` times; returns wall ms."""
    graph, gexec = C.c_void_p(), C.c_void_p()
    hip.check(hip.rt.hipStreamBeginCapture(stream, 2), "hipStreamBeginCapture")  # 2 = relaxed
    try:
        for i in range(per_graph):
            step(i)
    finally:
        rc = hip.rt.hipStreamEndCapture(stream, C.byref(graph))
    hip.check(rc, "hipStreamEndCapture")
    hip.check(hip.rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0), "hipGraphInstantiate")
    for _ in range(3):
        hip.check(hip.rt.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
    rnb.sync()
    t0 = time.perf_counter()
    for _ in range(n_graphs):
        hip.rt.hipGraphLaunch(gexec, stream)
    rnb.sync()
    ms = (time.perf_counter() - t0) * 1e3
    hip.rt.hipGraphExecDestroy(gexec)
    hip.rt.hipGraphDestroy(graph)
    return ms


# ---- algorithmic bytes (weights once + quantised activations once + f32 outputs once) --------------

def gemv_bytes(quant, rows, cols, seq=1):
    w = rows * (cols // BLOCK_ELEMS[quant]) * BLOCK_BYTES[quant]
    act = seq * (cols // 32 * 36 if quant == Q8_0 else cols // 256 * 292)
    return w + act + seq * rows * 4


def copies_for(nbytes):
    return max(2, -(-2 * MALL_BYTES // nbytes))


def one_launch_step(quant, rows, cols, seq):
    """True when the library runs the whole step (token quantisation + GEMV) as one kernel."""
    if seq != 1:
        return False
    if quant in (10, 11, Q4_K, Q5_K, Q6_K):
        nb = cols // 256
        return nb <= 64 and (nb <= 8 or rows * nb * BLOCK_BYTES.get(quant, 144) < (300 << 20))
    return cols // 32 <= 128 and rows * (cols // 32) >= 1 << 18


def bench_matmul(rnb, hip, stream, quant, rows, cols, seq, steps, warmup, seed, name, want_graph=True,
                 cache_resident=False, want_wall=True):
    w_host = synth_weights(quant, rows, cols, seed)
    n_copies = copies_for(w_host.nbytes)
    log(f"[{name}] weights {w_host.nbytes / 1e6:.1f} MB x {n_copies} device copies")
    w_dev = [rnb.DeviceBuffer.from_host(w_host) for _ in range(n_copies)]
    x = (np.random.default_rng(seed + 1).standard_normal(seq * cols)).astype(np.float32)
    x_dev = rnb.DeviceBuffer.from_host(x)
    out_dev = rnb.DeviceBuffer(seq * rows * 4)

    def step(i):
        rnb.gemv_dev(quant, w_dev[i % n_copies], rows, cols, x_dev, seq, out_dev)

    res = {"launch": "stream"}
    if want_wall:
        for i in range(warmup):
            step(i)
        wall_ms = wall_steps(rnb, step, steps)
        res["wall_ms_per_step"] = wall_ms / steps
    if want_graph:
        try:
            per = n_copies if steps >= n_copies else steps
            reps = max(1, steps // per)
            g_ms = graph_steps(hip, rnb, stream, step, per, reps)
            res["graph_ms_per_step"] = g_ms / (per * reps)
        except Exception as exc:  # keep the stream number if capture is unavailable
            log(f"[{name}] graph replay unavailable: {exc}")
    # the step as the library enqueues it (one launch, or activation quantiser + GEMV / GEMM [+ slice sum])
    res["step"] = kernel_stats(hip, stream, step)
    res["one_launch_step"] = one_launch_step(quant, rows, cols, seq)
    # the GEMV / GEMM alone over an already quantised activation
    rnb.quantize_dev(quant, x_dev, seq, cols)
    res["prequantised"] = kernel_stats(
        hip, stream, lambda i: rnb.gemv_quantized_dev(quant, w_dev[i % n_copies], rows, cols, seq, out_dev))
    if cache_resident:
        # one copy only: the weights may stay in the 256 MiB Infinity Cache; labelled, never `value`
        res["cache_resident"] = kernel_stats(hip, stream,
                                             lambda i: rnb.gemv_quantized_dev(quant, w_dev[0], rows, cols, seq, out_dev))
    res["bytes"] = gemv_bytes(quant, rows, cols, seq)
    res["copies"] = n_copies
    step(0)
    rnb.sync()
    out = out_dev.to_host(np.float32)
    for b in w_dev:
        b.free()
    x_dev.free()
    out_dev.free()
    return res, w_host, x, out


def _cpu_threads():
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    return min(threads, os.cpu_count() or threads)


CHECKS = []  # every GPU-vs-CPU comparison of this run: (leg, verdict); main() folds them into `all_checks_ok`


def _matches(leg, gpu, ref, flip_verdict=None):
    """GPU result against the CPU leg's: {"ok", "n_outside", "worst_over_tol", "flip_aware_ok"}.  The tolerance is the
    single-stage one, max(1e-3 * rms, 1e-3 * |ref|) per output.  Two-stage operators (MoE) pass `flip_verdict`, a
    function that decides whether outputs outside it differ by whole re-quantisation flips of the intermediate
    (oracle/flips.py); a leg that is neither `ok` nor `flip_aware_ok` is reported on stderr and fails the run."""
    e = np.asarray(ref, np.float64).ravel()
    g = np.asarray(gpu, np.float64).ravel()
    tol = np.maximum(1e-3 * np.sqrt(np.mean(e * e)), 1e-3 * np.abs(e))
    diff = np.abs(g - e)
    finite = bool(np.all(np.isfinite(g)))
    n_out = int(np.count_nonzero(diff > tol)) if finite else int(g.size)
    res = {"ok": bool(finite and n_out == 0), "n_outside": n_out,
           "worst_over_tol": float((diff / tol).max()) if finite else float("inf")}
    res["flip_aware_ok"] = res["ok"]
    if finite and n_out and flip_verdict is not None:
        res.update(flip_verdict())
    if not res["ok"]:
        log(f"CHECK {leg}: {n_out} of {g.size} outputs outside the plain tolerance (worst {res['worst_over_tol']:.2f} x tol); "
            + ("explained by re-quantisation flips: " + json.dumps(res.get("flips")) if res["flip_aware_ok"]
               else "NOT explained by re-quantisation flips: MISMATCH"))
    CHECKS.append((leg, res))
    return res


def cpu_baseline_gemv(quant, w_host, rows, cols, x, gpu_out, budget_s=10.0):
    """The CPU leg: rnb-cpu's x86 path restated in oracle/ (AVX2+FMA dots, contiguous row chunks per
    thread), timed on this host; also checks the GPU result against it (abs-or-rel 1e-3)."""
    from oracle import oracle as ora

    ora.lib()
    threads = _cpu_threads()
    avx2 = ora.have_avx2()
    run = lambda w: ora.gemv(quant, w, rows, cols, x, avx2=avx2, n_threads=threads)  # noqa: E731
    ref = run(w_host)
    # the scalar restatement on one thread, a few passes: sanity figure beside the threaded one
    t0 = time.perf_counter()
    n_scalar = 0
    while time.perf_counter() - t0 < 1.5:
        ora.gemv(quant, w_host, rows, cols, x, n_threads=1)
        n_scalar += 1
    scalar_ms = (time.perf_counter() - t0) / n_scalar * 1e3
    # the figure that is reported: the weights rotate over copies totalling more than the host's last-level caches,
    # as the GPU leg rotates over more than the Infinity Cache, for about `budget_s` seconds of CPU work
    n_copies = max(2, -(-(1 << 30) // max(1, w_host.nbytes)))
    copies = [w_host] + [w_host.copy() for _ in range(n_copies - 1)]
    for i in range(n_copies):  # thread pool and clocks warm before anything is timed
        run(copies[i])
    times, t_start, i = [], time.perf_counter(), 0
    while time.perf_counter() - t_start < budget_s:
        t0 = time.perf_counter()
        run(copies[i % n_copies])
        times.append(time.perf_counter() - t0)
        i += 1
    med = float(np.median(times))
    # one copy only, after the rotating loop (same warm threads): whatever the host caches keep of 33 MB
    single = []
    t_start = time.perf_counter()
    while len(single) < 200 and time.perf_counter() - t_start < 2.0:
        t0 = time.perf_counter()
        run(w_host)
        single.append(time.perf_counter() - t0)
    nbytes = gemv_bytes(quant, rows, cols, x.size // cols)
    return {"value": nbytes / med / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{len(times)} full passes of the same {rows}x{cols} GEMV over {n_copies} rotating weight copies "
                      f"({n_copies * w_host.nbytes / 1e6:.0f} MB, ~{budget_s:.0f} s of wall time), median per pass",
            "ms": med * 1e3, "single_copy_GB/s": nbytes / float(np.median(single)) / 1e9,
            "scalar_1_thread_ms": scalar_ms, "scalar_1_thread_GB/s": nbytes / scalar_ms / 1e6,
            "isa": "avx2+fma" if avx2 else "scalar", "gpu_matches_cpu": _matches(f"gemv quant {quant} {rows}x{cols}", gpu_out, ref),
            "note": "restatement of rnb-cpu's x86 path (Rust toolchain unavailable); a baseline, not a target"}


def cpu_baseline_gemm(w_host, rows, cols, x, gpu_out, sample_tokens=64, budget_s=12.0):
    """cfg4 on the CPU: the batch driver of crates/rnb-cpu/src/gemm/quant_gemv.rs:1127-1196 restated (rows chunked over
    threads, every row against every token), on the first `sample_tokens` of the 512 tokens; checks those tokens of the
    GPU result."""
    from oracle import oracle as ora

    ora.lib()
    threads = _cpu_threads()
    avx2 = ora.have_avx2()
    xs = np.ascontiguousarray(x[:sample_tokens * cols])
    run = lambda: ora.gemv(Q4_K, w_host, rows, cols, xs, avx2=avx2, n_threads=threads)  # noqa: E731
    ref = run()
    times, t_start = [], time.perf_counter()
    while time.perf_counter() - t_start < budget_s and len(times) < 50:
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    ops = 2 * sample_tokens * rows * cols
    got = np.asarray(gpu_out, np.float32).reshape(-1, rows)[:sample_tokens]
    return {"value": ops / med / 1e12, "unit": "TOP/s", "cores": threads, "kind": "port",
            "sample": f"{len(times)} passes over the first {sample_tokens} of the 512 tokens against all {rows} rows "
                      f"(an eighth of the workload per pass), median per pass", "ms": med * 1e3,
            "isa": "avx2+fma" if avx2 else "scalar", "gpu_matches_cpu": _matches("cfg4 gemm, first 64 tokens", got, ref)}


def bench_moe(rnb, hip, stream, tokens, steps, seed, cpu=True):
    n_expert, n_ff, n_embd, k = 128, 768, 2048, 8
    gen = 16  # distinct experts generated; tiled to 128 (addresses differ)
    per_gate = n_ff * (n_embd // 256) * 144
    per_down = n_embd * (n_ff // 256) * 210
    g = np.tile(synth_weights(Q4_K, gen * n_ff, n_embd, seed), n_expert // gen)
    u = np.tile(synth_weights(Q4_K, gen * n_ff, n_embd, seed + 1), n_expert // gen)
    d = np.tile(synth_weights(Q6_K, gen * n_embd, n_ff, seed + 2), n_expert // gen)
    gd, ud, dd = (rnb.DeviceBuffer.from_host(a) for a in (g, u, d))
    rng = np.random.default_rng(seed + 3)
    x_host = rng.standard_normal(tokens * n_embd).astype(np.float32)
    x_dev = rnb.DeviceBuffer.from_host(x_host)
    out_dev = rnb.DeviceBuffer(tokens * n_embd * 4)
    routes = []
    for it in range(8):  # the route changes per iteration, so 392 MB of experts are cycled through
        logits = rng.standard_normal((tokens, n_expert)).astype(np.float32)
        idx = np.argsort(-logits, axis=1, kind="stable")[:, :k]
        sel = np.take_along_axis(logits, idx, axis=1)
        wts = np.exp(sel - sel[:, :1])
        wts = (wts / wts.sum(axis=1, keepdims=True)).astype(np.float32)
        e = idx.reshape(-1).astype(np.uint32)
        t = np.repeat(np.arange(tokens, dtype=np.uint32), k)
        r = wts.reshape(-1)
        if tokens > 1:
            order = np.lexsort((t, e))
            e, t, r = e[order], t[order], r[order]
        routes.append((e, r, t))

    def step(i):
        e, r, t = routes[i % len(routes)]
        rnb.moe_sparse_experts_by_token_dev(gd, ud, dd, n_expert, e, r, t, tokens, Q6_K, n_ff, n_embd, x_dev, out_dev)

    st = kernel_stats(hip, stream, step)
    ms = st["mean"]
    distinct = float(np.mean([len(np.unique(rt[0])) for rt in routes]))
    weight_bytes = distinct * (2 * per_gate + per_down)
    nbytes = weight_bytes + tokens * k * 292 + tokens * n_embd * 4
    res = {"workload": f"cfg5 sparse MoE 128 experts top-8, hidden 2048, ffn 768, tokens={tokens}", "ms": ms,
           "ms_median": st["median"], "ms_p10": st["p10"], "ms_p90": st["p90"], "launches": st["launches"],
           "distinct_experts_mean": distinct, "bytes": nbytes, "GB/s": nbytes / ms / 1e6,
           "hbm_frac": nbytes / ms / 1e6 / HBM_PEAK_GBPS, "ops": 2 * tokens * k * 3 * n_ff * n_embd,
           "note": "events around the whole call (table upload + quantise + gate/up + re-quantise + down + reduce)"}
    if cpu:
        try:
            from oracle import oracle as ora

            ora.lib()
            threads = _cpu_threads()
            e, r, t = routes[0]
            step(0)
            rnb.sync()
            gpu_out = out_dev.to_host(np.float32)
            simd = ora.have_avx2()  # the timed form runs rnb-cpu's AVX2 block dots; the check uses the scalar form
            run = lambda rt, avx2=simd: ora.moe_sparse_experts_by_token(g, u, d, n_expert, rt[0], rt[1], rt[2], tokens,  # noqa: E731
                                                                        Q6_K, n_ff, n_embd, x_host, n_threads=threads,
                                                                        avx2=avx2)
            ref = run(routes[0], False)

            def flip_verdict():
                from oracle import flips

                v = flips.moe_verdict(gpu_out, ref, g, u, d, n_expert, e, r, t, tokens, Q6_K, n_ff, n_embd, x_host)
                return {key: v[key] for key in v if key not in ("ok", "n_outside", "worst_over_tol")}

            verdict = _matches(f"cfg5 moe tokens={tokens}", gpu_out, ref, flip_verdict)
            times, t_start, i = [], time.perf_counter(), 0
            while time.perf_counter() - t_start < 6.0 and len(times) < 200:
                t0 = time.perf_counter()
                run(routes[i % len(routes)])
                times.append(time.perf_counter() - t0)
                i += 1
            med = float(np.median(times))
            res["cpu_baseline"] = {"value": nbytes / med / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                                   "sample": f"{len(times)} full passes of the same routed call (routes rotate as on the GPU), "
                                             f"median per pass", "ms": med * 1e3, "gpu_matches_cpu": verdict,
                                   "note": "the per-token loop of prefill_cpu.rs:167-194 over the "
                                           + ("AVX2+FMA" if simd else "scalar") + " block dots, slots on threads; "
                                           "gpu_matches_cpu is taken against the scalar dots"}
        except Exception as exc:
            res["cpu_baseline"] = {"error": str(exc)}
    for b in (gd, ud, dd, x_dev, out_dev):
        b.free()
    return res


def bench_ffn(rnb, hip, stream, tokens, steps, seed):
    """Dense SwiGLU FFN of a Llama-3-8B layer through the device-resident operator: gate/up 14336x4096 Q4_K,
    down 4096x14336 Q6_K; the three matrices are rotated over enough copies to stream from HBM."""
    n_ff, n_embd = 14336, 4096
    g = synth_weights(Q4_K, n_ff, n_embd, seed)
    u = synth_weights(Q4_K, n_ff, n_embd, seed + 1)
    d = synth_weights(Q6_K, n_embd, n_ff, seed + 2)
    wbytes = g.nbytes + u.nbytes + d.nbytes
    n_copies = copies_for(wbytes)
    sets = [tuple(rnb.DeviceBuffer.from_host(a) for a in (g, u, d)) for _ in range(n_copies)]
    x_dev = rnb.DeviceBuffer.from_host(np.random.default_rng(seed + 3).standard_normal(tokens * n_embd).astype(np.float32))
    out_dev = rnb.DeviceBuffer(tokens * n_embd * 4)

    def step(i):
        gd, ud, dd = sets[i % n_copies]
        rnb.dense_q4k_silu_ffn_dev(gd, ud, dd, Q6_K, n_ff, n_embd, tokens, x_dev, out_dev)

    st = kernel_stats(hip, stream, step, launches=200 if tokens < 16 else 40, warmups=10, batch=10)
    ms = st["mean"]
    nbytes = wbytes + tokens * (n_embd // 256 * 292 + n_ff // 256 * 292 + n_embd * 4)
    for trio in sets:
        for b in trio:
            b.free()
    x_dev.free()
    out_dev.free()
    res = {"workload": f"dense SwiGLU FFN 4096 -> 14336 -> 4096 (Q4_K gate/up, Q6_K down), tokens={tokens}", "ms": ms,
           "ms_median": st["median"], "ms_p10": st["p10"], "ms_p90": st["p90"], "launches": st["launches"], "copies": n_copies}
    if tokens < 16:  # decode: weight streaming
        res.update({"bytes": nbytes, "GB/s": nbytes / ms / 1e6, "hbm_frac": nbytes / ms / 1e6 / HBM_PEAK_GBPS,
                    "note": "events around the whole call (token quantisation + gate/up/SiLU in one launch, re-quantise, down)"})
    else:  # prefill: matrix-core GEMMs
        ops = 2 * tokens * 3 * n_ff * n_embd
        res.update({"ops": ops, "TOP/s": ops / ms / 1e9, "mfma_frac": ops / ms / 1e9 / INT8_PEAK_TOPS,
                    "note": "events around the whole call (quantise, two Q4_K GEMMs, SiLU*up quantised as it is made, Q6_K GEMM)"})
    return res


# configs that --only can run alone: quant, rows, cols, tokens
ONLY = {"cfg1": (Q8_0, 4096, 4096, 1), "cfg2": (Q4_K, 14336, 4096, 1), "cfg3a": (Q6_K, 4096, 14336, 1),
        "cfg3b": (Q6_K, 128256, 4096, 1), "cfg4": (Q4_K, 14336, 4096, 512), "q6gemm": (Q6_K, 4096, 14336, 512), "q5gemm": (Q5_K, 14336, 4096, 512),
        "moe1": 1, "moe4": 4, "moe64": 64,  # moeN: configs[4] at N tokens
        "ffn1": 1, "ffn512": 512}  # ffnN: the dense Llama-3-8B FFN at N tokens


def run_only(rnb, hip, stream, name, calibration):
    """One config, 60 steps after 10 warm-ups (plus the calibration copies when asked): what a counter run profiles."""
    if calibration:
        calibration_copy(hip, rnb, stream)
    if name.startswith("moe"):
        res = bench_moe(rnb, hip, stream, ONLY[name], 0, 1234 + ONLY[name], cpu=False)
        print(json.dumps({"only": name, "step_ms_median": res["ms_median"], "launches": res["launches"]}), flush=True)
        return 0
    if name.startswith("ffn"):
        res = bench_ffn(rnb, hip, stream, ONLY[name], 0, 4321)
        print(json.dumps({"only": name, "step_ms_median": res["ms_median"], "launches": res["launches"]}), flush=True)
        return 0
    quant, rows, cols, seq = ONLY[name]
    w_host = synth_weights(quant, rows, cols, 20240607)
    n_copies = copies_for(w_host.nbytes)
    w_dev = [rnb.DeviceBuffer.from_host(w_host) for _ in range(n_copies)]
    x_dev = rnb.DeviceBuffer.from_host(np.random.default_rng(1).standard_normal(seq * cols).astype(np.float32))
    out_dev = rnb.DeviceBuffer(seq * rows * 4)
    st = kernel_stats(hip, stream, lambda i: rnb.gemv_dev(quant, w_dev[i % n_copies], rows, cols, x_dev, seq, out_dev),
                      launches=60, warmups=10, batch=10)
    print(json.dumps({"only": name, "step_ms_median": st["median"], "launches": st["launches"], "copies": n_copies}), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--quick", action="store_true", help="headline config only (skip the secondary configs)")
    ap.add_argument("--only", choices=sorted(ONLY), help="one config's step, a few dozen launches, for counter runs under "
                                                         "rocprofv3 --pmc (prints a short JSON line of its own)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a 64 MiB device-to-device copy (reference for FETCH_SIZE / WRITE_SIZE under --pmc)")
    ap.add_argument("--cache-resident", action="store_true",
                    help="also time each kernel on ONE weight copy (may be served by the Infinity Cache)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures the single-GPU hot path only: every box in this build has one GPU, and the path "
            "has no collectives (it shards by weight rows / by expert). Run with --gpus 1.")
        return 2

    import runnburn_amd as rnb  # raises when librnb_hip.so has not been built: no fallback

    if not rnb.device_available():
        log(f"no MI355X device: {rnb.last_error()}")
        return 3
    hip = Hip()
    stream = C.c_void_p(rnb.stream_handle())
    log(f"device: {rnb.device_name()}")

    if args.only:
        return run_only(rnb, hip, stream, args.only, args.calibration_copy)
    if args.calibration_copy:
        calibration_copy(hip, rnb, stream)
    rows, cols = 14336, 4096
    main_res, w_host, x, gpu_out = bench_matmul(rnb, hip, stream, Q4_K, rows, cols, 1, args.steps, args.warmup, 20240607,
                                                "cfg2 q4k gemv", cache_resident=args.cache_resident)
    nbytes = main_res["bytes"]
    step_ms = min(main_res["wall_ms_per_step"], main_res.get("graph_ms_per_step", float("inf")))
    launch = "graph" if main_res.get("graph_ms_per_step", float("inf")) <= main_res["wall_ms_per_step"] else "stream"
    kst = main_res["step"]
    achieved = nbytes / kst["mean"] / 1e6
    result = {
        "metric": "Q4_K decode GEMV HBM GB/s (% of 8 TB/s); prefill GEMM TOPS (% MFMA)",
        "value": nbytes / step_ms / 1e6,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u4 x i8 -> i32, f32 scales",
        "data": "synthetic, seeded: fp32 N(0,0.02) weights fitted to valid GGUF blocks by a vectorised numpy min/max fit "
                "inside bench.py (not the restated ggml quantiser: kernel speed does not depend on the values), fp32 N(0,1) "
                "activations",
        "config": {"workload": "configs[1]: Q4_K decode GEMV, weights 14336x4096 (Llama-3-8B FFN up/gate), 1 token, "
                               "step = device Q8_K quantisation + GEMV (one launch)", "rows": rows, "cols": cols, "tokens": 1,
                   "weight_copies_rotated": main_res["copies"], "step_launch": launch,
                   "stream_ms_per_step": main_res["wall_ms_per_step"],
                   "graph_ms_per_step": main_res.get("graph_ms_per_step")},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": measured_traffic("gemv_kquant_f32_kernel<12,1>"),
                     "traffic_source": "not measured in this run: the committed counter summary "
                                       "profiles/gemv_q4k_cfg2_hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE "
                                       "of this kernel on this workload, each scaled by the calibration copy's reading)",
                     "kernel": "gemv_kquant_f32_kernel<12,1> (Q8_K quantisation of the token + GEMV in one launch)",
                     "bytes_per_launch": nbytes, "kernel_ms_mean": kst["mean"], "kernel_ms_median": kst["median"],
                     "kernel_ms_p10": kst["p10"], "kernel_ms_p90": kst["p90"], "launches": kst["launches"],
                     "warmup_launches": kst["warmups"],
                     "prequantised_gemv_kernel_ms_median": main_res["prequantised"]["median"],
                     "timing": "HIP events on the library stream: 200 back-to-back launches after 20 warm-ups, an event every "
                               "10 launches; mean over all, median / p10 / p90 over the batches"},
    }
    try:  # what a kernel that only reads reaches in this run: on the headline's bytes and on cfg3b's
        result["roofline"]["read_ceiling"] = read_ceiling(hip, rnb, stream, 33030144)
        result["roofline"]["read_ceiling_431MB"] = read_ceiling(hip, rnb, stream, 430940160)
    except Exception as exc:
        log(f"read ceiling skipped: {exc}")
    try:  # what the runtime's own device copy reaches on the same number of bytes, for context
        result["roofline"]["device_copy_same_size"] = copy_context(hip, rnb, stream, 33030144)
    except Exception as exc:
        log(f"copy context skipped: {exc}")
    if "cache_resident" in main_res:
        result["roofline"]["cache_resident_GBps"] = nbytes / main_res["cache_resident"]["median"] / 1e6
    if not args.no_cpu_baseline:
        try:
            result["cpu_baseline"] = cpu_baseline_gemv(Q4_K, w_host, rows, cols, x, gpu_out)
        except Exception as exc:
            log(f"cpu baseline failed: {exc}")
            result["cpu_baseline"] = None
    del w_host

    # ---- the metric's second half: cfg4, Q4_K prefill GEMM, 512 tokens x 4096 -> 14336 -----------------------------
    try:
        res4, w4, x4, out4 = bench_matmul(rnb, hip, stream, Q4_K, 14336, 4096, 512, 40, 5, 99, "cfg4 q4k gemm",
                                          want_graph=False, want_wall=False)
        ops = 2 * 512 * 14336 * 4096
        pq = res4["prequantised"]
        tops = ops / pq["mean"] / 1e9
        result["roofline_gemm"] = {
            "bound": "mfma", "achieved": tops, "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": tops / INT8_PEAK_TOPS,
            "traffic": None, "workload": "configs[3]: Q4_K prefill GEMM, 512 tokens x 4096 -> 14336",
            "kernel": "gemm_q4k_mfma_kernel (Q4_K x Q8_K on v_mfma_i32_32x32x32_i8)", "ops_per_launch": ops,
            "kernel_ms_mean": pq["mean"], "kernel_ms_median": pq["median"], "kernel_ms_p10": pq["p10"],
            "kernel_ms_p90": pq["p90"], "launches": pq["launches"],
            "step_ms_median": res4["step"]["median"], "step": "activation quantiser (512 x 4096 f32 -> Q8_K) + GEMM"}
        try:
            result["roofline_gemm"]["mfma_ceiling"] = mfma_ceiling(hip, rnb, stream)
        except Exception as exc:
            log(f"mfma ceiling skipped: {exc}")
        if not args.no_cpu_baseline:
            try:
                result["cpu_baseline_gemm"] = cpu_baseline_gemm(w4, 14336, 4096, x4, out4)
            except Exception as exc:
                log(f"cpu baseline (gemm) failed: {exc}")
                result["cpu_baseline_gemm"] = None
        del w4, x4, out4
    except Exception as exc:
        result["roofline_gemm"] = {"error": str(exc)}

    if not args.quick:
        sec = {}
        s2 = max(50, min(args.steps, 500))
        for key, quant, r, c, seq in (("cfg1_q8_0_gemv_4096x4096", Q8_0, 4096, 4096, 1),
                                      ("cfg3a_q6k_gemv_4096x14336", Q6_K, 4096, 14336, 1),
                                      ("cfg3b_q6k_gemv_128256x4096", Q6_K, 128256, 4096, 1),
                                      ("q5k_gemv_14336x4096", Q5_K, 14336, 4096, 1)):
            try:
                res, _, _, _ = bench_matmul(rnb, hip, stream, quant, r, c, seq, s2, 10, 7 + r, key, want_graph=False,
                                            cache_resident=args.cache_resident, want_wall=False)
                st, pq = res["step"], res["prequantised"]
                gbps = res["bytes"] / st["mean"] / 1e6
                sec[key] = {"step_ms_mean": st["mean"], "step_ms_median": st["median"], "step_ms_p10": st["p10"],
                            "step_ms_p90": st["p90"], "launches": st["launches"], "bytes": res["bytes"], "GB/s": gbps,
                            "hbm_frac": gbps / HBM_PEAK_GBPS, "copies": res["copies"],
                            "step": "one launch: token quantisation + GEMV" if res["one_launch_step"]
                            else "two launches: activation quantiser, then the GEMV",
                            "prequantised_gemv_ms_median": pq["median"],
                            "prequantised_gemv_GB/s": res["bytes"] / pq["median"] / 1e6}
                if "cache_resident" in res:
                    sec[key]["cache_resident_GB/s"] = res["bytes"] / res["cache_resident"]["median"] / 1e6
            except Exception as exc:
                sec[key] = {"error": str(exc)}
        # prefill on the formats whose scales cannot ride on an int8 operand (scale groups applied on the vector units)
        for key, quant, r, c in (("q6k_gemm_512x14336_to_4096", Q6_K, 4096, 14336), ("q5k_gemm_512x4096_to_14336", Q5_K, 14336, 4096),
                                 ("q8_0_gemm_512x4096_to_4096", Q8_0, 4096, 4096)):
            try:
                res, _, _, _ = bench_matmul(rnb, hip, stream, quant, r, c, 512, 20, 3, 101, key, want_graph=False,
                                            want_wall=False)
                ops = 2 * 512 * r * c
                pq = res["prequantised"]
                tops = ops / pq["mean"] / 1e9
                sec[key] = {"kernel_ms_mean": pq["mean"], "kernel_ms_median": pq["median"], "kernel_ms_p10": pq["p10"],
                            "kernel_ms_p90": pq["p90"], "ops": ops, "TOP/s": tops, "mfma_frac": tops / INT8_PEAK_TOPS}
            except Exception as exc:
                sec[key] = {"error": str(exc)}
        # small batches (several sequences decoding together): the GEMV that keeps four tokens in registers per pass
        try:
            res, _, _, _ = bench_matmul(rnb, hip, stream, Q4_K, 14336, 4096, 4, s2, 10, 7 + 4, "q4k 14336x4096 x 4 tokens",
                                        want_graph=False, want_wall=False)
            st = res["step"]
            sec["q4k_14336x4096_tokens4"] = {"step_ms_mean": st["mean"], "step_ms_median": st["median"], "step_ms_p10": st["p10"],
                                             "step_ms_p90": st["p90"], "launches": st["launches"],
                                             "step": "two launches: activation quantiser, then one pass over the matrix for "
                                                     "the four tokens"}
        except Exception as exc:
            sec["q4k_14336x4096_tokens4"] = {"error": str(exc)}
        for tokens in (1, 4, 64):
            try:
                sec[f"cfg5_moe_tokens{tokens}"] = bench_moe(rnb, hip, stream, tokens, s2, 1234 + tokens,
                                                            cpu=not args.no_cpu_baseline)
            except Exception as exc:
                sec[f"cfg5_moe_tokens{tokens}"] = {"error": str(exc)}
        for tokens, n in ((1, s2), (512, 20)):
            try:
                sec[f"ffn_llama3_8b_tokens{tokens}"] = bench_ffn(rnb, hip, stream, tokens, n, 4321)
            except Exception as exc:
                sec[f"ffn_llama3_8b_tokens{tokens}"] = {"error": str(exc)}
        result["secondary"] = sec

    # every comparison with the CPU legs, folded: plain tolerance, or (two-stage operators) whole re-quantisation flips
    result["all_checks_ok"] = bool(CHECKS) and all(v["ok"] or v["flip_aware_ok"] for _, v in CHECKS)
    result["checks"] = {leg: ("ok" if v["ok"] else "flips" if v["flip_aware_ok"] else "MISMATCH") for leg, v in CHECKS}
    if args.no_cpu_baseline:
        result["all_checks_ok"] = None  # nothing was compared
    print(json.dumps(result), flush=True)
    if result["all_checks_ok"] is False:
        log("bench.py: a GPU result does not match its CPU leg; see the CHECK lines above")
        return 4
    return 0


if __name__ == "__main__":
    sys.exit(main())
