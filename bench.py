#!/usr/bin/env python3
"""Headline benchmark of the Matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (BASELINE.json configs[1]): Q8_0 GEMV, Phi-2 decode MLP up-projection:
x [1 x 2560] f16, W [10240 x 2560] Q8_0H in the reference's segment layout,
f16 bias [10240], called as W.gemm(x, bias, false, true, true).  One step is
one such GEMV.  The weight is replicated into enough distinct device copies
that their footprint exceeds the 256 MB Infinity Cache, and successive steps
rotate over them, so every step streams its weight from HBM.  All inputs are
resident in HBM before the timed region; nothing is copied or allocated inside
it.

Prints one JSON line.  `value` is algorithmic bytes per step / mean time per
step over the timed region (HIP events on the launch stream).  `roofline`
prices the same figure against the 8 TB/s HBM peak, `cpu_baseline` is the CPU
oracle (dequantize -> f32 GEMV -> bias -> cast) timed on the host cores of the
same machine, and `secondary` reports the other BASELINE shapes the same way.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense f16 matrix peak
INFINITY_CACHE_BYTES = 256 << 20

# HBM bytes per launch of the GEMV kernel from two rocprofv3 --pmc runs (FETCH_SIZE, then
# WRITE_SIZE, each scaled by what the same counter reads for a 256 MiB copy); the commands and
# readings are in profiles/gemv_q8_phi2_m1_pmc.txt.  A counter reading cannot be taken inside
# this script, so the figure is the recorded one for the M=1 workload.  The readings were taken on
# the build whose gemv_q8h_rowdot_kernel / gemm_nt_dl_kernel sources are the ones in this tree
# (git log -- ratchet_amd/csrc/kernels_gemv.hip ratchet_amd/csrc/kernels_gemm_nt.hip names the
# last change to each); a change to either kernel's loads or stores needs the two --pmc runs again.
GEMV_TRAFFIC_BYTES = 27985470
# The same for the f16 GEMM of the metric's second half (profiles/gemm_c4_f16_q8_pmc.txt): FETCH_SIZE
# 36,025 KiB x 1.99982 (copy calibration) + WRITE_SIZE 11,531 KiB.  The weight is read once and the
# activations once per XCD (eight L2s), which is what puts it above the 65.6 MB the shape holds.
GEMM_F16_TRAFFIC_BYTES = 85580611


def gemv_bytes(M, N, K):
    """Algorithmic bytes of one Q8_0H Linear: int8 weights + f16 scales + x + bias + y."""
    return N * K + (N * K // 32) * 2 + M * K * 2 + N * 2 + M * N * 2


class Runner:
    """Enqueues pre-built descriptors through the C ABI on torch's current stream."""

    def __init__(self):
        import torch

        from ratchet_amd import Device, DeviceRequest, _ffi
        self.torch, self.ffi = torch, _ffi
        self.dev = Device.request_device(DeviceRequest.GPU)
        self.L = _ffi.lib()

    def upload(self, arr: np.ndarray):
        t = self.torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1).copy())
        return t.to("cuda:0")

    def workspace(self, desc):
        """Device memory with which the library cuts this product along K, or None when it would not."""
        need = ctypes.c_uint64()
        st = self.L.rt_matmul_workspace_bytes(self.dev.ctx, ctypes.byref(desc), ctypes.byref(need))
        if st != self.ffi.RT_OK:
            raise RuntimeError(f"rt_matmul_workspace_bytes: {self.ffi.status_string(st)}")
        return self.torch.empty(need.value, dtype=self.torch.uint8, device="cuda:0") if need.value else None

    def enqueue(self, desc, lhs, rhs, bias, out, act=0, ws=None):
        st = self.L.rt_matmul_enqueue_ws(
            self.dev.ctx, ctypes.byref(desc), ctypes.c_void_p(lhs.data_ptr()), ctypes.c_void_p(rhs.data_ptr()),
            ctypes.c_void_p(bias.data_ptr()) if bias is not None else None, ctypes.c_void_p(out.data_ptr()), act,
            ctypes.c_void_p(ws.data_ptr()) if ws is not None else None, ws.numel() if ws is not None else 0,
            ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream))
        if st != self.ffi.RT_OK:
            raise RuntimeError(f"rt_matmul_enqueue: {self.ffi.status_string(st)} "
                               f"{self.L.rt_last_error(self.dev.ctx).decode()}")

    REGIONS = 11   # timed regions of `steps` launches each; the median is reported

    def wall_clock_ms_per_step(self, launch_step, n_variants, replays=2000):
        """A cross-check of the event timing that uses no HIP event: `replays` replays of a HIP graph of one
        rotation of the weight copies (20 launches or more) between two device synchronisations, timed with the
        host's clock.  The host enqueues a replay much faster than the device runs it, so the device is never idle
        in between; the figure includes the ends of the replays (about 0.2 us per launch more than launches that
        follow each other in a stream)."""
        torch = self.torch
        per_graph = n_variants * -(-20 // n_variants)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(per_graph):
                launch_step(i % n_variants)
        for _ in range(10):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / (replays * per_graph), replays * per_graph

    MAX_COVER = 256  # untimed graph replays the host may put in front of a region to stay ahead of the device

    def time_steps(self, launch_step, steps, warmup, n_variants, stats=None):
        """Times `steps` calls of launch_step(i) after `warmup` untimed ones, REGIONS times over, each region
        between its own pair of HIP events on the launch stream, and returns the median region's
        (ms_per_step, mode); `stats`, a dict, also receives the fastest and slowest region and the count.

        The host needs longer to enqueue a launch than a ~6 us kernel runs, so a region must not contain the
        host's enqueue time.  The launches are captured once into a HIP graph of whole rotations of the weight
        copies (20 launches or more).  Two kinds of region:
          "stream behind a hipgraph cover": untimed replays of that graph keep the device busy while the host
              enqueues the first event, the `steps` launches one by one as any caller would, and the second
              event; by the time the cover has drained, the host is far enough ahead that the device never waits
              for it: a region counts only if the device still had a backlog when the last launch had been
              enqueued, else all regions are taken again behind twice the cover.  Used when at most MAX_COVER
              replays give that head start (any kernel of a few microseconds or more).
          "hipgraph": otherwise (kernels much shorter than an enqueue) the region is steps // 20 replays of the
              graph plus the remaining launches one by one, behind one untimed replay.  Launches inside a
              replay follow each other about 0.2 us more slowly than launches in a stream, and a replay adds
              about 5 us at its start and end.
        Without graph capture all launches are issued one by one."""
        torch = self.torch
        for i in range(warmup):
            launch_step(i % n_variants)
        torch.cuda.synchronize()
        mode, graph, covers = "stream", None, 0
        per_graph = n_variants * -(-20 // n_variants)  # at least 20 launches per replay
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(per_graph):
                    launch_step(i % n_variants)
            graph.replay()
            torch.cuda.synchronize()
            mode = "hipgraph"
        except Exception as e:  # capture refused: fall back to plain launches
            sys.stderr.write(f"bench: graph capture unavailable ({type(e).__name__}: {e}); plain launches\n")
            graph = None
            torch.cuda.synchronize()
        if graph is not None:
            # what the host needs per enqueue and the device per step: the cover must outlast the difference
            t0 = time.perf_counter()
            for i in range(per_graph):
                launch_step(i % n_variants)
            host_s = (time.perf_counter() - t0) / per_graph
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            graph.replay()
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            dev_s = e0.elapsed_time(e1) * 1e-3 / per_graph
            covers = 1 + int(-(-max(0.0, steps * (1.5 * host_s - dev_s) + 100e-6) // (per_graph * dev_s)))

        def region(covers):
            """One timed region: (ms per step, seconds the device still had to run when the host had enqueued it all)."""
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            if covers:
                for _ in range(covers):
                    graph.replay()
                e0.record()
                for i in range(steps):
                    launch_step(i % n_variants)
            elif graph is not None:
                graph.replay()  # the device is still busy with it while the host enqueues the event and the timed replays
                e0.record()
                full, rest = divmod(steps, per_graph)
                for _ in range(full):
                    graph.replay()
                for i in range(rest):
                    launch_step(i % n_variants)
            else:
                e0.record()
                for i in range(steps):
                    launch_step(i % n_variants)
            e1.record()
            t_enq = time.perf_counter()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / steps, time.perf_counter() - t_enq

        # A covered region counts only if the device was still well behind the host when the last launch had been
        # enqueued (the backlog shrinks all the way through a region, so then it never ran dry).  If one was not,
        # all regions are taken again behind twice the cover; past MAX_COVER the graph replays are timed instead.
        times = []
        while graph is not None and covers:
            if covers > self.MAX_COVER:
                covers = 0
                break
            runs = [region(covers) for _ in range(self.REGIONS)]
            if all(backlog >= max(200e-6, 10 * dev_s) for _, backlog in runs):
                times, mode = [ms for ms, _ in runs], "stream behind a hipgraph cover"
                break
            covers *= 2
        if not times:
            times = [region(0)[0] for _ in range(self.REGIONS)]
        times.sort()
        if stats is not None:
            stats.update(regions=len(times), ms_per_step_min=times[0], ms_per_step_max=times[-1], cover_replays=covers)
        return times[len(times) // 2], mode


def bench_q8_gemv(r: Runner, O, M, steps, warmup, seed=0, copies=None, wall_clock=False):
    """C2.  `copies` = 1 measures the warm case (the one weight stays in the 256 MB Infinity Cache); the
    default rotates enough copies that every launch streams its weight from HBM."""
    N, K = 10240, 2560
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    wbuf = O.make_q8_0h(w)
    x = rng.standard_normal((1, M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    per = gemv_bytes(M, N, K)
    if copies is None:
        copies = max(2, -(-2 * INFINITY_CACHE_BYTES // wbuf.size))  # footprint >= 2x the Infinity Cache
    ws = [r.upload(wbuf) for _ in range(copies)]
    xd, bd = r.upload(x), r.upload(bias)
    outs = [r.torch.empty(M * N * 2, dtype=r.torch.uint8, device="cuda:0") for _ in range(copies)]
    desc = r.ffi.make_desc(r.ffi.RT_Q8_0H, (N, K), r.ffi.RT_F16, (1, M, K), False, True, True, r.ffi.RT_F16, (N,))
    stats = {}
    ms, mode = r.time_steps(lambda i: r.enqueue(desc, ws[i], xd, bd, outs[i]), steps, warmup, copies, stats)
    if wall_clock:
        stats["wall_clock_ms_per_step"], stats["wall_clock_launches"] = r.wall_clock_ms_per_step(
            lambda i: r.enqueue(desc, ws[i], xd, bd, outs[i]), copies)
    # parity of what was just timed, against the oracle on the same inputs
    got = outs[(steps - 1) % copies].cpu().numpy().view(np.float16).reshape(1, M, N)
    ref = O.matmul_ref(wbuf, O.Q8_0H, (N, K), x, O.F16, x.shape, bias, False, True, True)
    err = O.max_rel_err(got, ref)
    if not err <= 2e-2:
        raise RuntimeError(f"bench output differs from the oracle: max_rel_err={err}")
    return dict(ms=ms, bytes=per, gbps=per / (ms * 1e-3) / 1e9, mode=mode, copies=copies, err=err,
                inputs=(wbuf, x, bias), stats=stats)


def bench_q8_gemm(r: Runner, O, steps, warmup, act=0):
    """C4 up-projection: X [512 x 2560] f16 . W[10240 x 2560]^T Q8_0H + bias (MFMA-bound); with
    `act` the GELU that follows it in the model (phi2/mlp.rs:13-15) runs in the same kernel."""
    M, N, K = 512, 10240, 2560
    rng = np.random.default_rng(4)
    wbuf = O.make_q8_0h((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    x = rng.standard_normal((1, M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    wd, xd, bd = r.upload(wbuf), r.upload(x), r.upload(bias)
    out = r.torch.empty(M * N * 2, dtype=r.torch.uint8, device="cuda:0")
    desc = r.ffi.make_desc(r.ffi.RT_Q8_0H, (N, K), r.ffi.RT_F16, (1, M, K), False, True, True, r.ffi.RT_F16, (N,))
    ms, mode = r.time_steps(lambda i: r.enqueue(desc, wd, xd, bd, out, act), steps, warmup, 1)
    flops = 2.0 * M * N * K
    if act:  # the first rows against the oracle's fused statement
        got = out.cpu().numpy().view(np.float16).reshape(1, M, N)[:, :16]
        ref = O.matmul_ref(wbuf, O.Q8_0H, (N, K), x[:, :16], O.F16, (1, 16, K), bias, False, True, True, act=act)
        err = O.max_rel_err(got, ref)
        if not err <= 2e-2:
            raise RuntimeError(f"fused Q8_0H GEMM output differs from the oracle: max_rel_err={err}")
    return dict(workload="C4 up: X[512x2560] f16 . Q8_0H W[10240x2560]^T + bias" + (", GELU fused" if act else ""), ms=ms,
                tflops=flops / (ms * 1e-3) / 1e12, mode=mode)


def bench_f16_gemm(r: Runner, O, steps, warmup, M=512):
    """The C4 shape with plain f16 weights: X [512 x 2560] . W[10240 x 2560]^T + bias (the f16 GEMM headline).
    Larger M (more activation rows against the same weight) shows what the kernel does when the shape is not
    the limit: at 512 rows the grid is exactly one workgroup per compute unit."""
    N, K = 10240, 2560
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    x = rng.standard_normal((1, M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    wd, xd, bd = r.upload(w), r.upload(x), r.upload(bias)
    out = r.torch.empty(M * N * 2, dtype=r.torch.uint8, device="cuda:0")
    desc = r.ffi.make_desc(r.ffi.RT_F16, (N, K), r.ffi.RT_F16, (1, M, K), False, True, True, r.ffi.RT_F16, (N,))
    ms, mode = r.time_steps(lambda i: r.enqueue(desc, wd, xd, bd, out), steps, warmup, 1)
    got = out.cpu().numpy().view(np.float16).reshape(M, N)[:64]
    ref = x[0, :64].astype(np.float64) @ w.astype(np.float64).T + bias.astype(np.float64)
    err = O.max_rel_err(got, ref)
    if not err <= 2e-2:
        raise RuntimeError(f"f16 GEMM output differs from float64: max_rel_err={err}")
    return dict(workload=f"C4 shape, f16 weights: X[{M}x2560] f16 . W[10240x2560]^T f16 + bias", ms=ms,
                tflops=2.0 * M * N * K / (ms * 1e-3) / 1e12, mode=mode, flops=2.0 * M * N * K,
                bytes=2 * (M * K + N * K + N + M * N))


def bench_generic(r: Runner, O, name, lhs, lhs_dt, lhs_shape, rhs, rhs_shape, bias, flags, act, flops, nbytes, steps,
                  tol, split_k=False):
    """Any other BASELINE shape: time it, check it against the oracle on its first stack rows.
    `split_k` hands the launch the workspace the library asks for (rt_matmul_workspace_bytes)."""
    ffi = r.ffi
    act_dt = ffi.RT_F16 if act == np.float16 else ffi.RT_F32
    ridge = (157.3e12 if act == np.float32 else MFMA_F16_PEAK_TFLOPS * 1e12) / (HBM_PEAK_GBPS * 1e9)
    hbm_bound = flops / nbytes <= ridge
    # below the ridge point the operands are rotated over a footprint of 2x the Infinity Cache
    copies = max(2, -(-2 * INFINITY_CACHE_BYTES // (lhs.nbytes + rhs.nbytes))) if hbm_bound else 1
    lds, rds = [r.upload(lhs) for _ in range(copies)], [r.upload(rhs) for _ in range(copies)]
    bd = None if bias is None else r.upload(bias)
    desc = ffi.make_desc(lhs_dt, lhs_shape, act_dt, rhs_shape, *flags,
                         None if bias is None else act_dt, None if bias is None else bias.shape)
    oshape = (ctypes.c_int64 * ffi.RT_MAX_RANK)()
    orank, odt = ctypes.c_int32(), ctypes.c_int32()
    r.L.rt_matmul_infer(ctypes.byref(desc), oshape, ctypes.byref(orank), ctypes.byref(odt))
    oshape = tuple(oshape[i] for i in range(orank.value))
    outs = [r.torch.empty(int(np.prod(oshape)) * np.dtype(act).itemsize, dtype=r.torch.uint8, device="cuda:0")
            for _ in range(copies)]
    ws = r.workspace(desc) if split_k else None
    ms, mode = r.time_steps(lambda i: r.enqueue(desc, lds[i], rds[i], bd, outs[i], 0, ws), steps, 5, copies)
    got = outs[-1].cpu().numpy().view(act).reshape(oshape)
    odt_id = {ffi.RT_F32: O.F32, ffi.RT_F16: O.F16, ffi.RT_Q8_0F: O.Q8_0F, ffi.RT_Q8_0H: O.Q8_0H, ffi.RT_Q4_K: O.Q4_K}
    t0 = time.perf_counter()
    ref = O.matmul_ref(lhs, odt_id[lhs_dt], lhs_shape, rhs, odt_id[act_dt], rhs_shape, bias, *flags)
    cpu_ms = (time.perf_counter() - t0) * 1e3   # the oracle's path on the host cores, one run, same inputs
    err = O.max_rel_err(got, ref)
    if not err <= tol:
        raise RuntimeError(f"{name}: output differs from the oracle: max_rel_err={err}")
    d = {"workload": name, "ms_per_step": ms}
    if split_k:
        d["workspace_bytes"] = 0 if ws is None else ws.numel()
    d.update(copies=copies, timing=mode, cpu_oracle_ms=round(cpu_ms, 2), cpu_threads=O.lib().orc_num_threads())
    if not hbm_bound:   # above the ridge point: price against the matrix peak
        d.update(value=round(flops / (ms * 1e-3) / 1e12, 1), unit="TFLOP/s")
    else:
        d.update(value=round(nbytes / (ms * 1e-3) / 1e9, 1), unit="GB/s",
                 frac_hbm_peak=round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4))
    return d


def bench_softmax(r: Runner, O):
    """The step between C3's two matmuls: in-place softmax of the f32 scores [32 x 512 x 512]
    (callers upcast the scores to f32, phi3/attn.rs:153).  One read and one write of the tensor."""
    ffi = r.ffi
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((1, 32, 512, 512)) * 2).astype(np.float32)
    copies = max(2, -(-2 * INFINITY_CACHE_BYTES // x.nbytes))
    xs = [r.upload(x) for _ in range(copies)]
    shape = (ctypes.c_int64 * ffi.RT_MAX_RANK)(*x.shape)

    def step(i):
        st = r.L.rt_softmax_enqueue(r.dev.ctx, ffi.RT_F32, ctypes.c_void_p(xs[i].data_ptr()), 4, shape, 3,
                                      ctypes.c_void_p(r.torch.cuda.current_stream().cuda_stream))
        if st != ffi.RT_OK:
            raise RuntimeError(f"rt_softmax_enqueue: {ffi.status_string(st)}")

    step(0)  # checked on the first application; later ones re-normalise their own output
    r.torch.cuda.synchronize()
    got = xs[0].cpu().numpy().view(np.float32).reshape(x.shape)
    t0 = time.perf_counter()
    ref = O.softmax(x)
    cpu_ms = (time.perf_counter() - t0) * 1e3
    if not np.allclose(got, ref, rtol=1e-5, atol=1e-6):
        raise RuntimeError("softmax: output differs from the oracle")
    ms, mode = r.time_steps(step, 200, 5, copies)
    nbytes = 2 * x.nbytes
    return {"workload": "C3 softmax f32 [32x512x512], in place", "ms_per_step": ms, "copies": copies, "timing": mode,
            "cpu_oracle_ms": round(cpu_ms, 2), "cpu_threads": O.lib().orc_num_threads(),
            "value": round(nbytes / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
            "frac_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}


def bench_elementwise(r: Runner, O):
    """The operators a model runs on C4's [512 x 10240] f16 activations when they are not fused:
    GELU (ops/unary.rs) and the casts around attention (ops/cast.rs).  One read and one write."""
    ffi, out = r.ffi, []
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((512, 10240)) * 2).astype(np.float16)
    copies = max(2, -(-2 * INFINITY_CACHE_BYTES // (3 * x.nbytes)))
    xs = [r.upload(x) for _ in range(copies)]
    ys = [r.torch.empty(x.size * 4, dtype=r.torch.uint8, device="cuda:0") for _ in range(copies)]
    stream = lambda: ctypes.c_void_p(r.torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def check(st):
        if st != ffi.RT_OK:
            raise RuntimeError(f"elementwise enqueue: {ffi.status_string(st)} {r.L.rt_last_error(r.dev.ctx).decode()}")

    def gelu(i):
        check(r.L.rt_unary_enqueue(r.dev.ctx, ffi.RT_ACT_GELU, ffi.RT_F16, p(xs[i]), p(ys[i]), x.size, stream()))

    def widen(i):
        check(r.L.rt_cast_enqueue(r.dev.ctx, ffi.RT_F16, ffi.RT_F32, p(xs[i]), p(ys[i]), x.size, stream()))

    for name, step, nbytes, ref, view in (
            ("GELU f16 [512x10240] (unfused operator)", gelu, 2 * x.nbytes, lambda: O.unary(x, O.ACT_GELU), np.float16),
            ("cast f16 -> f32 [512x10240]", widen, 3 * x.nbytes, lambda: O.cast(x, np.float32), np.float32)):
        step(copies - 1)
        r.torch.cuda.synchronize()
        got = ys[copies - 1].cpu().numpy().view(view)[: x.size].reshape(x.shape)
        t0 = time.perf_counter()
        want = ref()
        cpu_ms = (time.perf_counter() - t0) * 1e3
        if not np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=1e-3, atol=1e-6):
            raise RuntimeError(f"{name}: output differs from the oracle")
        ms, mode = r.time_steps(step, 200, 5, copies)
        out.append({"workload": name, "ms_per_step": ms, "copies": copies, "timing": mode,
                    "cpu_oracle_ms": round(cpu_ms, 2), "cpu_threads": O.lib().orc_num_threads(),
                    "value": round(nbytes / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                    "frac_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
    return out


def bench_attention(r: Runner, O):
    """C3 as one kernel: softmax(q k^T / sqrt(80)) v for 32 heads x 512 x 80 (prefill), and one decode
    step against 2048 cached keys.  Algorithmic bytes: q, k, v read once, out written once."""
    ffi, out = r.ffi, []
    for name, Lq, Lk, causal, reps in (("C3 fused attention f16 [32x512x80], prefill", 512, 512, 0, 200),
                                       ("C3 fused attention f16 [32x512x80], causal prefill", 512, 512, 1, 200),
                                       ("attention decode step: 1 query x 2048 cached keys, 32 heads x 80", 1, 2048, 1, 200)):
        rng = np.random.default_rng(7)
        B, H, D = 1, 32, 80
        q = rng.standard_normal((B, H, Lq, D)).astype(np.float16)
        k = rng.standard_normal((B, H, Lk, D)).astype(np.float16)
        v = rng.standard_normal((B, H, Lk, D)).astype(np.float16)
        nbytes = 2 * q.nbytes + k.nbytes + v.nbytes
        copies = max(2, -(-2 * INFINITY_CACHE_BYTES // nbytes))
        qs, ks, vs = ([r.upload(a) for _ in range(copies)] for a in (q, k, v))
        outs = [r.torch.empty(q.nbytes, dtype=r.torch.uint8, device="cuda:0") for _ in range(copies)]
        d = ffi.AttentionDesc()
        d.dtype, d.batch, d.heads, d.q_len, d.kv_len, d.head_dim = ffi.RT_F16, B, H, Lq, Lk, D
        d.q_strides[:] = [H * Lq * D, Lq * D, D]
        d.o_strides[:] = [H * Lq * D, Lq * D, D]
        d.k_strides[:] = [H * Lk * D, Lk * D, D]
        d.v_strides[:] = [H * Lk * D, Lk * D, D]
        d.scale, d.causal, d.mask_dtype, d.mask_row_stride = float(1 / np.sqrt(D)), causal, ffi.RT_F32, Lk
        p = lambda t: ctypes.c_void_p(t.data_ptr())

        need = ctypes.c_uint64()
        r.L.rt_attention_workspace_bytes(ctypes.byref(d), ctypes.byref(need))
        ws = r.torch.empty(max(need.value, 16), dtype=r.torch.uint8, device="cuda:0")

        def step(i):
            st = r.L.rt_attention_enqueue(r.dev.ctx, ctypes.byref(d), p(qs[i]), p(ks[i]), p(vs[i]), None, p(outs[i]),
                                          p(ws), need.value, ctypes.c_void_p(r.torch.cuda.current_stream().cuda_stream))
            if st != ffi.RT_OK:
                raise RuntimeError(f"rt_attention_enqueue: {ffi.status_string(st)} {r.L.rt_last_error(r.dev.ctx).decode()}")

        step(copies - 1)
        r.torch.cuda.synchronize()
        got = outs[copies - 1].cpu().numpy().view(np.float16).reshape(q.shape)
        t0 = time.perf_counter()
        ref = O.attention(q[:, :4], k[:, :4], v[:, :4], causal=bool(causal))   # the first four heads
        cpu_ms = (time.perf_counter() - t0) * 1e3 * (H / 4)
        if not np.allclose(got[:, :4].astype(np.float32), ref.astype(np.float32), rtol=2e-2, atol=2e-3):
            raise RuntimeError(f"{name}: output differs from the oracle")
        ms, mode = r.time_steps(step, reps, 5, copies)
        flops = 4.0 * B * H * Lq * Lk * D * (0.5 if causal and Lq == Lk else 1.0)
        out.append({"workload": name, "ms_per_step": ms, "copies": copies, "timing": mode,
                    "cpu_oracle_ms": round(cpu_ms, 2), "cpu_threads": O.lib().orc_num_threads(),
                    "value": round(nbytes / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                    "frac_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "tflops": round(flops / (ms * 1e-3) / 1e12, 1)})
    return out


def bench_decoder_layer(r: Runner, O, kv_len=1024, layers=8, fused_qkv=False):
    """One decode step of the two blocks of a Phi-2 decoder layer that this library's operators cover
    (crates/ratchet-models/src/phi2/attn.rs, mlp.rs; no normalisation, rotary embedding or residual adds):
    q, k, v projections (3 GEMVs), two cache writes, attention over `kv_len` cached keys read in place,
    output projection, fc1 with GELU fused, fc2.  Nine launches per layer; `layers` distinct layers
    (Q8_0H weights, 83.6 MB each) are chained in one graph so that no weight is served from cache.
    `fused_qkv`: the q, k and v weights are one [7680 x 2560] tensor, concatenated when the model is loaded (the
    layout the reference's Phi-3 ships with, phi3/attn.rs:55,95-108), so the three projections are one launch whose
    output the cache writes and the attention read in place through strides."""
    ffi, torch = r.ffi, r.torch
    W, H, D, HID, cap = 2560, 32, 80, 10240, 2048
    rng = np.random.default_rng(8)
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def linear(n, k, upload=True):
        w = (rng.standard_normal((n, k)) * (1.0 / np.sqrt(k))).astype(np.float32)
        b = (rng.standard_normal(n) * 0.05).astype(np.float16)
        q = O.make_q8_0h(w)
        return (r.upload(q) if upload else None), r.upload(b), q, w, b

    mods = []
    for li in range(layers):
        keep_host = li == layers - 1   # only the checked layer's host copies are kept
        m = {name: linear(n, k, not (fused_qkv and name in "qkv")) for name, (n, k) in
             {"q": (W, W), "k": (W, W), "v": (W, W), "o": (W, W), "fc1": (HID, W), "fc2": (W, HID)}.items()}
        if fused_qkv:
            # blocks of 32 never straddle rows, so the concatenation's blocks are the three tensors' blocks
            m["qkv"] = (r.upload(O.make_q8_0h(np.concatenate([m[n][3] for n in "qkv"]))),
                        r.upload(np.concatenate([m[n][4] for n in "qkv"])))
        for n in list(m):
            if n != "qkv":
                m[n] = m[n][:3] if keep_host else (m[n][0], m[n][1], None)
        m["kc"] = r.upload((rng.standard_normal((1, H, cap, D)) * 0.5).astype(np.float16))
        m["vc"] = r.upload((rng.standard_normal((1, H, cap, D)) * 0.5).astype(np.float16))
        mods.append(m)
    x = rng.standard_normal((1, 1, W)).astype(np.float16)
    xd = r.upload(x)
    buf = {n: torch.empty(sz * 2, dtype=torch.uint8, device="cuda:0") for n, sz in
           {"q": W, "k": W, "v": W, "qkv": 3 * W, "a": W, "o": W, "h": HID, "y": W}.items()}
    desc = lambda n, k: ffi.make_desc(ffi.RT_Q8_0H, (n, k), ffi.RT_F16, (1, 1, k), False, True, True, ffi.RT_F16, (n,))
    d_ww, d_hw, d_wh, d_3w = desc(W, W), desc(HID, W), desc(W, HID), desc(3 * W, W)
    QW = 3 * W if fused_qkv else W         # row stride of the projections' output
    ad = ffi.AttentionDesc()
    ad.dtype, ad.batch, ad.heads, ad.q_len, ad.kv_len, ad.head_dim = ffi.RT_F16, 1, H, 1, kv_len, D
    ad.q_strides[:] = [QW, D, QW]          # q as the projection leaves it: [1, 1, heads * d]
    ad.o_strides[:] = [W, D, W]            # and the result the same way
    ad.k_strides[:] = [H * cap * D, cap * D, D]
    ad.v_strides[:] = [H * cap * D, cap * D, D]
    ad.scale, ad.causal, ad.mask_dtype, ad.mask_row_stride = float(1 / np.sqrt(D)), 1, ffi.RT_F32, kv_len
    sstr = (ctypes.c_int64 * 3)(QW, D, QW)
    off = lambda t, halfs: ctypes.c_void_p(t.data_ptr() + 2 * halfs)
    need = ctypes.c_uint64()
    r.L.rt_attention_workspace_bytes(ctypes.byref(ad), ctypes.byref(need))
    ws = torch.empty(max(need.value, 16), dtype=torch.uint8, device="cuda:0")

    def check(st, what):
        if st != ffi.RT_OK:
            raise RuntimeError(f"{what}: {ffi.status_string(st)} {r.L.rt_last_error(r.dev.ctx).decode()}")

    def layer(m):
        if fused_qkv:
            r.enqueue(d_3w, m["qkv"][0], xd, m["qkv"][1], buf["qkv"])
            qp, kp, vp = p(buf["qkv"]), off(buf["qkv"], W), off(buf["qkv"], 2 * W)
        else:
            for n in ("q", "k", "v"):
                r.enqueue(d_ww, m[n][0], xd, m[n][1], buf[n])
            qp, kp, vp = p(buf["q"]), p(buf["k"]), p(buf["v"])
        if fused_qkv:   # both caches by one launch
            check(r.L.rt_cache_write_kv_enqueue(r.dev.ctx, ffi.RT_F16, p(m["kc"]), kp, p(m["vc"]), vp, sstr, 1, H, cap,
                                                kv_len - 1, 1, D, stream()), "cache write")
        else:
            for c, src in (("kc", kp), ("vc", vp)):
                check(r.L.rt_cache_write_enqueue(r.dev.ctx, ffi.RT_F16, p(m[c]), src, sstr, None, 1, H, cap, kv_len - 1, 1, D,
                                                 stream()), "cache write")
        check(r.L.rt_attention_enqueue(r.dev.ctx, ctypes.byref(ad), qp, p(m["kc"]), p(m["vc"]), None, p(buf["a"]),
                                       p(ws), need.value, stream()), "attention")
        r.enqueue(d_ww, m["o"][0], buf["a"], m["o"][1], buf["o"])
        r.enqueue(d_hw, m["fc1"][0], xd, m["fc1"][1], buf["h"], ffi.RT_ACT_GELU)
        r.enqueue(d_wh, m["fc2"][0], buf["h"], m["fc2"][1], buf["y"])

    # check the last layer's two outputs against the oracle's composition
    layer(mods[-1])
    torch.cuda.synchronize()
    m = mods[-1]
    lin = lambda n, xin, shape, act=0: O.matmul_ref(m[n][2], O.Q8_0H, shape, xin, O.F16, xin.shape,
                                                     m[n][1].cpu().numpy().view(np.float16), False, True, True, act=act)
    t0 = time.perf_counter()
    y_ref = lin("fc2", lin("fc1", x, (HID, W), O.ACT_GELU), (W, HID))
    qh, kh, vh = (lin(n, x, (W, W)).reshape(1, 1, H, D).transpose(0, 2, 1, 3) for n in ("q", "k", "v"))
    kc = m["kc"].cpu().numpy().view(np.float16).reshape(1, H, cap, D)[:, :, :kv_len]
    vc = m["vc"].cpu().numpy().view(np.float16).reshape(1, H, cap, D)[:, :, :kv_len]
    a_ref = O.attention(qh, kc, vc, causal=True).transpose(0, 2, 1, 3).reshape(1, 1, W)
    o_ref = lin("o", a_ref, (W, W))
    cpu_ms = (time.perf_counter() - t0) * 1e3
    got_y = buf["y"].cpu().numpy().view(np.float16).reshape(1, 1, W)
    got_o = buf["o"].cpu().numpy().view(np.float16).reshape(1, 1, W)
    if not (O.max_rel_err(got_y, y_ref) <= 2e-2 and np.allclose(got_o.astype(np.float32), o_ref.astype(np.float32), rtol=2e-2, atol=4e-3)):
        raise RuntimeError("decoder layer: output differs from the oracle's composition")
    near = lambda a, b_: np.allclose(a.astype(np.float32), b_.astype(np.float32), rtol=2e-2, atol=4e-3)
    if not (near(kc[:, :, kv_len - 1], kh[:, :, 0]) and near(vc[:, :, kv_len - 1], vh[:, :, 0])):
        raise RuntimeError("decoder layer: the cache does not hold the new key / value")
    ms, mode = r.time_steps(lambda i: layer(mods[i]), 200, 5, layers)
    wbytes = sum(m[n][0].numel() + m[n][1].numel() for n in (("qkv",) if fused_qkv else ("q", "k", "v")) + ("o", "fc1", "fc2"))
    nbytes = wbytes + 2 * H * kv_len * D * 2
    what = "q/k/v weights concatenated at load and one launch for both cache writes, 6 launches" if fused_qkv else "9 launches"
    return {"workload": f"Phi-2 decoder layer decode step (attention block + MLP, Q8_0H, {kv_len} cached keys), {what}",
            "ms_per_step": ms, "copies": layers, "timing": mode, "cpu_oracle_ms": round(cpu_ms, 2),
            "cpu_threads": O.lib().orc_num_threads(), "value": round(nbytes / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
            "frac_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "layers_per_second": round(1e3 / ms, 1)}


def other_configs(r: Runner, O):
    """The matmul shapes of the other benchmark configurations (Whisper encoder f32 GEMM, attention
    products at 32 heads x 512 x 80, Q4_K projections): algorithmic flops and bytes are spelled out per call."""
    ffi, out = r.ffi, []
    rng = np.random.default_rng(0)
    a = (rng.standard_normal((1500, 384)) * 0.05).astype(np.float32)
    b = (rng.standard_normal((384, 1536)) * 0.05).astype(np.float32)
    bias = (rng.standard_normal(1536) * 0.05).astype(np.float32)
    out.append(bench_generic(r, O, "C1 f32 GEMM [1500x384].[384x1536]+b", a, ffi.RT_F32, a.shape, b, b.shape, bias,
                             (False, False, False), np.float32, 1769472000, 13885440, 200, 1e-3))
    out += c3_products(r, O)
    # the C2 shape with unquantized weights (the reference's GEMV kernels serve f32, f16 and Q8_0: ops/gemv.rs:156-574;
    # Quantization::F16 / F32 checkpoints of Phi-2 decode through these)
    rng = np.random.default_rng(7)
    w = (rng.standard_normal((10240, 2560)) * 0.02).astype(np.float32)
    x = rng.standard_normal((1, 1, 2560)).astype(np.float32)
    bias = rng.standard_normal(10240).astype(np.float32)
    for name, dt, cast, tol in (("f16", ffi.RT_F16, np.float16, 2e-2), ("f32", ffi.RT_F32, np.float32, 1e-3)):
        wb, xb, bb = w.astype(cast), x.astype(cast), bias.astype(cast)
        out.append(bench_generic(r, O, f"C2 shape, {name} weights: x[1x2560] . W[10240x2560]^T + bias, M=1", wb, dt, wb.shape, xb,
                                 xb.shape, bb, (False, True, True), cast, 2.0 * 10240 * 2560,
                                 (10240 * 2560 + 2560 + 2 * 10240) * wb.itemsize, 200, tol))
    # the Phi-2 down-projection with f16 weights: rows of 20 KiB (the looping form of the row-streaming kernel)
    w = (rng.standard_normal((2560, 10240)) * 0.02).astype(np.float16)
    x = rng.standard_normal((1, 1, 10240)).astype(np.float16)
    bias = rng.standard_normal(2560).astype(np.float16)
    out.append(bench_generic(r, O, "down-projection shape, f16 weights: x[1x10240] . W[2560x10240]^T + bias, M=1", w, ffi.RT_F16, w.shape,
                             x, x.shape, bias, (False, True, True), np.float16, 2.0 * 2560 * 10240,
                             (2560 * 10240 + 10240 + 2 * 2560) * 2, 200, 2e-2))
    # C4's second half: the down-projection has 64 output tiles and K = 10240; with the workspace the
    # library asks for, its K is cut among four workgroups per tile (rt_matmul_enqueue_ws)
    rng = np.random.default_rng(6)
    w = (rng.standard_normal((2560, 10240)) * 0.02).astype(np.float32)
    x = rng.standard_normal((1, 512, 10240)).astype(np.float16)
    bias = rng.standard_normal(2560).astype(np.float16)
    for name, lhs, dt, wbytes in (("f16", w.astype(np.float16), ffi.RT_F16, 2560 * 10240 * 2),
                                  ("Q8_0H", O.make_q8_0h(w), ffi.RT_Q8_0H, 2560 * 10240 * 17 // 16)):
        out.append(bench_generic(r, O, f"C4 down: X[512x10240] f16 . {name} W[2560x10240]^T + bias, K split with a workspace",
                                 lhs, dt, (2560, 10240), x, x.shape, bias, (False, True, True), np.float16,
                                 2.0 * 512 * 2560 * 10240, wbytes + (512 * 10240 + 2560 + 512 * 2560) * 2, 50, 2e-2,
                                 split_k=True))
    out.append(bench_softmax(r, O))
    out += bench_attention(r, O)
    out.append(bench_decoder_layer(r, O))
    out.append(bench_decoder_layer(r, O, fused_qkv=True))
    out += bench_q4k(r, O, (1, 16, 128, 256), 200)
    # short prompts against the C4 up-projection, the weights from HBM: 16 / 32 / 64 rows on the weight-streaming
    # GEMM (Q8_0H at 16 rows on the streaming GEMV, at 64 on 64-row tiles), 128 rows on 64-row weight tiles so that
    # every compute unit has a workgroup (160 workgroups; the 160-row tile would leave 64)
    rng = np.random.default_rng(8)
    w = (rng.standard_normal((10240, 2560)) * 0.02).astype(np.float32)
    bias = rng.standard_normal(10240).astype(np.float16)
    for rows in (16, 32, 64, 128):
        x = rng.standard_normal((1, rows, 2560)).astype(np.float16)
        for name, lhs, dt, wbytes in (("f16", w.astype(np.float16), ffi.RT_F16, 10240 * 2560 * 2),
                                      ("Q8_0H", O.make_q8_0h(w), ffi.RT_Q8_0H, 10240 * 2560 * 17 // 16)):
            out.append(bench_generic(r, O, f"C4 up at {rows} rows: X[{rows}x2560] f16 . {name} W[10240x2560]^T + bias", lhs, dt,
                                     (10240, 2560), x, x.shape, bias, (False, True, True), np.float16, 2.0 * rows * 10240 * 2560,
                                     wbytes + (rows * 2560 + 10240 + rows * 10240) * 2, 100, 2e-2))
    return out


def c3_products(r: Runner, O):
    """BASELINE configs[2]: the two attention products at 32 heads x 512 x 80, f16, and the f32 spelling of the first."""
    ffi, out = r.ffi, []
    rng = np.random.default_rng(1)
    q = rng.standard_normal((1, 32, 512, 80)).astype(np.float16)
    k = rng.standard_normal((1, 32, 512, 80)).astype(np.float16)
    v = rng.standard_normal((1, 32, 512, 80)).astype(np.float16)
    p = (rng.random((1, 32, 512, 512)) / 512).astype(np.float16)
    out.append(bench_generic(r, O, "C3 QK^T f16 [32x512x80].[32x512x80]^T", q, ffi.RT_F16, q.shape, k, k.shape, None,
                             (False, True, False), np.float16, 1342177280, 22020096, 200, 2e-2))
    out.append(bench_generic(r, O, "C3 PV f16 [32x512x512].[32x512x80]", p, ffi.RT_F16, p.shape, v, v.shape, None,
                             (False, False, False), np.float16, 1342177280, 22020096, 200, 2e-2))
    # the phi2 / whisper spelling of the score product: f32 operands, the key permuted beforehand, matmul(false, false)
    # (crates/ratchet-models/src/phi2/attn.rs:139-142): reads 2 x 5.2 MB, writes 33.6 MB of f32 scores
    qf, ktf = q.astype(np.float32), np.ascontiguousarray(k.astype(np.float32).transpose(0, 1, 3, 2))
    out.append(bench_generic(r, O, "C3 QK^T f32, key permuted beforehand [32x512x80].[32x80x512]", qf, ffi.RT_F32, qf.shape, ktf,
                             ktf.shape, None, (False, False, False), np.float32, 1342177280, 2 * 5242880 + 33554432, 200, 1e-3))
    return out


def bench_q4k(r: Runner, O, rows, steps):
    """BASELINE configs[4]: Q4_K W[8192x3072] against 1 / 16 (streaming kernel) and 128 / 256 (tiled kernel) f16 rows."""
    ffi, out = r.ffi, []
    rng = np.random.default_rng(5)
    blocks = O.q4k_quantize((rng.standard_normal((8192, 3072)) * 0.02).astype(np.float32))
    for M in rows:
        x = rng.standard_normal((1, M, 3072)).astype(np.float16)
        out.append(bench_generic(r, O, f"C5 Q4_K M={M} x[{M}x3072].W[8192x3072]^T", blocks, ffi.RT_Q4_K, (8192, 3072), x,
                                 x.shape, None, (False, True, True), np.float16, 50331648 * M,
                                 14155776 + 6144 * M + 16384 * M, steps, 2e-2))
    # a down-projection with K = 8192 (Phi-3-mini's, phi3/mlp.rs): rows of 32 super-blocks, one vector
    blocks = O.q4k_quantize((rng.standard_normal((3072, 8192)) * 0.02).astype(np.float32))
    x = rng.standard_normal((1, 1, 8192)).astype(np.float16)
    out.append(bench_generic(r, O, "Q4_K M=1, K = 8192: x[1x8192].W[3072x8192]^T", blocks, ffi.RT_Q4_K, (3072, 8192), x, x.shape,
                             None, (False, True, True), np.float16, 2.0 * 3072 * 8192, 3072 * 32 * 144 + 2 * 8192 + 2 * 3072, steps, 2e-2))
    return out


def read_calibration(r: Runner, O, steps, warmup):
    """Context for the headline: on the same 20 rotated copies of the 27.85 MB weight and with the same graph
    timing, what a launch costs that does nothing, what one costs that only reads the buffer (consecutive
    addresses, with and without non-temporal loads; the same with four bytes stored per wavefront, as the GEMV
    stores its results: a kernel that leaves modified lines in the L2s pays for their write-back when it ends; and
    in the 16-row pattern the matrix-core kernel reads it in), and the GEMV itself.  The probes are in ratchet_amd/libratchet_probes.so (csrc/bench_probes.hip)."""
    N, K = 10240, 2560
    rng = np.random.default_rng(0)
    wbuf = O.make_q8_0h((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    copies = max(2, -(-2 * INFINITY_CACHE_BYTES // wbuf.size))
    ws = [r.upload(wbuf) for _ in range(copies)]
    sink = r.torch.zeros(4096, dtype=r.torch.uint8, device="cuda:0")
    P = ctypes.CDLL(os.path.join(ROOT, "ratchet_amd", "libratchet_probes.so"))
    vp, u64, i64 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int64
    P.probe_empty.argtypes, P.probe_read_linear.argtypes = [vp, vp], [vp, u64, ctypes.c_int, vp, vp]
    P.probe_read_rows16.argtypes = [vp, i64, i64, vp, vp]
    P.probe_read_linear_store.argtypes = [vp, u64, vp, vp]
    stream = lambda: vp(r.torch.cuda.current_stream().cuda_stream)
    nbytes = wbuf.size - wbuf.size % 16

    def ok(rc):
        if rc != 0:
            raise RuntimeError(f"probe launch failed: hipError {rc}")

    x = rng.standard_normal((1, 1, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    xd, bd = r.upload(x), r.upload(bias)
    out = r.torch.empty(N * 2, dtype=r.torch.uint8, device="cuda:0")
    store_out = r.torch.empty(4 * 4 * (-(-nbytes // 5120 // 4) + 1), dtype=r.torch.uint8, device="cuda:0")  # whole workgroups of 4
    desc = r.ffi.make_desc(r.ffi.RT_Q8_0H, (N, K), r.ffi.RT_F16, (1, 1, K), False, True, True, r.ffi.RT_F16, (N,))
    lib_src = [w[:nbytes].view(r.torch.float32) for w in ws]
    lib_dst = r.torch.empty_like(lib_src[0])
    lib_sum = lambda i: r.torch.sum(lib_src[i])
    lib_mat = [w[:10240 * 1360 * 2].view(r.torch.float16).view(10240, 1360) for w in ws]
    lib_vec = r.torch.ones(1360, dtype=r.torch.float16, device="cuda:0")
    lib_mv = lambda i: r.torch.mv(lib_mat[i], lib_vec)
    rows = []
    for name, step, nb in (
            ("empty kernel (one wavefront)", lambda i: ok(P.probe_empty(vp(sink.data_ptr()), stream())), 0),
            ("read only, consecutive addresses", lambda i: ok(P.probe_read_linear(vp(ws[i].data_ptr()), nbytes, 0, vp(sink.data_ptr()), stream())), nbytes),
            ("read only, consecutive addresses, non-temporal loads", lambda i: ok(P.probe_read_linear(vp(ws[i].data_ptr()), nbytes, 1, vp(sink.data_ptr()), stream())), nbytes),
            ("read (non-temporal) + 4 bytes stored per wavefront of 5 KiB", lambda i: ok(P.probe_read_linear_store(vp(ws[i].data_ptr()), nbytes, vp(store_out.data_ptr()), stream())), nbytes),
            # passes over the same bytes by kernels this repository did not write: torch's reduction, the vendor BLAS's
            # GEMV reading the buffer as an f16 [10240 x 1360] matrix, the runtime's device copy (reads and writes)
            ("library: torch.sum over the weight as f32 (read only)", lambda i: lib_sum(i), nbytes),
            ("library: torch.mv, the weight as f16 [10240 x 1360] (vendor BLAS GEMV, read only)", lambda i: lib_mv(i), 10240 * 1360 * 2),
            ("library: device-to-device copy of the weight (reads and writes the bytes)", lambda i: lib_dst.copy_(lib_src[i], non_blocking=True), 2 * nbytes),
            ("read only, 16 rows x 64 bytes per load (the int8 codes alone)", lambda i: ok(P.probe_read_rows16(vp(ws[i].data_ptr()), N, K, vp(sink.data_ptr()), stream())), N * K),
            ("Q8_0H GEMV M=1 (the headline)", lambda i: r.enqueue(desc, ws[i], xd, bd, out), gemv_bytes(1, N, K))):
        stats = {}
        ms, mode = r.time_steps(step, steps, warmup, copies, stats)
        rows.append({"launch": name, "us_per_launch": round(ms * 1e3, 3), "us_min": round(stats["ms_per_step_min"] * 1e3, 3),
                     "bytes": nb, "GB/s": round(nb / (ms * 1e-3) / 1e9, 1) if nb else None, "timing": mode})
    return {"read_calibration": rows, "weight_copies_rotated": copies, "steps": steps, "regions": Runner.REGIONS}


def issue_calibration(r: Runner):
    """Context for the tiled kernels that decode or fold in their multiplying wavefronts: what MFMAs, packed vector
    instructions and LDS fragment reads cost a wavefront alone and mixed.  One wavefront per SIMD on every compute
    unit runs 4000 trips of (8 MFMAs, 8 x NV packed FMAs, ND fragment reads); ns per trip from HIP events around
    one launch, median of 5.  The probe is in ratchet_amd/libratchet_probes.so (csrc/bench_probes.hip)."""
    torch = r.torch
    P = ctypes.CDLL(os.path.join(ROOT, "ratchet_amd", "libratchet_probes.so"))
    vp = ctypes.c_void_p
    P.probe_issue_mix.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, vp]
    src = torch.zeros(8192, dtype=torch.uint8, device="cuda:0")
    dst = torch.zeros(256 * 1024, dtype=torch.uint8, device="cuda:0")
    iters, rows = 4000, []
    mixes = [("8 MFMAs", 0, 8, 0, 0), ("24 packed FMAs", 3, 0, 0, 0), ("8 MFMAs + 8 packed FMAs", 1, 8, 0, 0),
             ("8 MFMAs + 16 packed FMAs", 2, 8, 0, 0), ("8 MFMAs + 24 packed FMAs", 3, 8, 0, 0),
             ("8 MFMAs + 32 packed FMAs", 4, 8, 0, 0), ("8 MFMAs + 48 packed FMAs", 6, 8, 0, 0),
             ("8 MFMAs + 4 fragment reads", 0, 8, 4, 0), ("24 packed FMAs + 4 fragment reads", 3, 0, 4, 0),
             ("8 MFMAs + 24 packed FMAs + 2 fragment reads, each in front of an MFMA", 3, 8, 2, 0),
             ("8 MFMAs + 24 packed FMAs + 4 fragment reads, each in front of an MFMA", 3, 8, 4, 0),
             ("8 MFMAs + 24 packed FMAs + 8 fragment reads, each in front of an MFMA", 3, 8, 8, 0),
             ("8 MFMAs + 24 packed FMAs + 4 fragment reads, each right behind an MFMA", 3, 8, 4, 1),
             ("8 MFMAs + 24 packed FMAs + 8 fragment reads, each right behind an MFMA", 3, 8, 8, 1)]
    for name, nv, nm, nd, behind in mixes:
        def launch():
            rc = P.probe_issue_mix(nv, nm, nd, behind, iters, vp(src.data_ptr()), vp(dst.data_ptr()), vp(torch.cuda.current_stream().cuda_stream))
            if rc != 0:
                raise RuntimeError(f"probe launch failed: hipError {rc}")
        launch()
        torch.cuda.synchronize()
        ts = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            launch()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e6 / iters)
        ts.sort()
        rows.append({"trip": name, "ns_per_trip": round(ts[2], 1)})
    return {"issue_calibration": rows, "trips": iters, "wavefronts_per_simd": 1}


def host_enqueue_cost(r: Runner, O, calls=2000):
    """Host microseconds per enqueue of the headline GEMV through rt_matmul_enqueue_ws (guards, shape rules and
    lowering on every call) and through a plan (rt_matmul_plan_create once, rt_matmul_plan_enqueue per call): `calls`
    back-to-back calls from a C++ loop in ratchet_amd/libratchet_probes.so, host steady clock, no Python in the loop."""
    N, K = 10240, 2560
    rng = np.random.default_rng(0)
    wd = r.upload(O.make_q8_0h((rng.standard_normal((N, K)) * 0.02).astype(np.float32)))
    xd, bd = r.upload(rng.standard_normal((1, 1, K)).astype(np.float16)), r.upload(rng.standard_normal(N).astype(np.float16))
    out = r.torch.empty(N * 2, dtype=r.torch.uint8, device="cuda:0")
    desc = r.ffi.make_desc(r.ffi.RT_Q8_0H, (N, K), r.ffi.RT_F16, (1, 1, K), False, True, True, r.ffi.RT_F16, (N,))
    P = ctypes.CDLL(os.path.join(ROOT, "ratchet_amd", "libratchet_probes.so"))
    vp = ctypes.c_void_p
    P.probe_host_ns_enqueue_ws.restype = P.probe_host_ns_plan_enqueue.restype = ctypes.c_double
    P.probe_host_ns_enqueue_ws.argtypes = [vp, vp, vp, vp, vp, vp, vp, ctypes.c_int32, vp, ctypes.c_int]
    P.probe_host_ns_plan_enqueue.argtypes = [vp, vp, vp, vp, vp, vp, vp, ctypes.c_int]
    addr = lambda name: ctypes.cast(getattr(r.L, name), vp)
    stream = vp(r.torch.cuda.current_stream().cuda_stream)
    plan = vp()
    if r.L.rt_matmul_plan_create(r.dev.ctx, ctypes.byref(desc), 0, ctypes.byref(plan)) != r.ffi.RT_OK:
        raise RuntimeError("rt_matmul_plan_create failed")
    res = {}
    try:
        for _ in range(2):  # the first pass warms the code paths
            a = P.probe_host_ns_enqueue_ws(addr("rt_matmul_enqueue_ws"), r.dev.ctx, ctypes.byref(desc), vp(wd.data_ptr()), vp(xd.data_ptr()),
                                           vp(bd.data_ptr()), vp(out.data_ptr()), 0, stream, calls)
            r.torch.cuda.synchronize()
            b = P.probe_host_ns_plan_enqueue(addr("rt_matmul_plan_enqueue"), plan, vp(wd.data_ptr()), vp(xd.data_ptr()), vp(bd.data_ptr()),
                                             vp(out.data_ptr()), stream, calls)
            r.torch.cuda.synchronize()
        if a < 0 or b < 0:
            raise RuntimeError("an enqueue failed inside the host-cost probe")
        res = {"rt_matmul_enqueue_ws": round(a * 1e-3, 3), "rt_matmul_plan_enqueue": round(b * 1e-3, 3), "calls": calls,
               "how": "back-to-back calls from a C++ loop (no Python), host steady clock, launches piling up on the stream"}
    finally:
        r.L.rt_matmul_plan_destroy(plan)
    return res


def gemm_ablation(r: Runner):
    """What bounds the f16 tiled GEMM at X[512 x 2560] . W[10240 x 2560]^T + bias: the shipped kernel next to timing-only
    builds of the same source with parts left out (their results are wrong; ratchet_amd/libratchet_probes.so holds them,
    built from csrc/kernels_gemm_nt.hip with RT_NT_ABLATION set).  Same timing as every other workload here."""
    torch = r.torch
    M, N, K = 512, 10240, 2560
    rng = np.random.default_rng(5)
    wd = r.upload((rng.standard_normal((N, K)) * 0.02).astype(np.float16))
    xd = r.upload(rng.standard_normal((1, M, K)).astype(np.float16))
    bd = r.upload(rng.standard_normal(N).astype(np.float16))
    out = torch.empty(M * N * 2, dtype=torch.uint8, device="cuda:0")
    desc = r.ffi.make_desc(r.ffi.RT_F16, (N, K), r.ffi.RT_F16, (1, M, K), False, True, True, r.ffi.RT_F16, (N,))
    P = ctypes.CDLL(os.path.join(ROOT, "ratchet_amd", "libratchet_probes.so"))
    vp, i64 = ctypes.c_void_p, ctypes.c_int64

    def variant(mask):
        fn = getattr(P, f"probe_gemm_nt_ablation_{mask}")
        fn.argtypes = [vp, vp, vp, vp, i64, i64, i64, vp]

        def step(i):
            rc = fn(vp(wd.data_ptr()), vp(xd.data_ptr()), vp(bd.data_ptr()), vp(out.data_ptr()), N, M, K,
                    vp(torch.cuda.current_stream().cuda_stream))
            if rc != 0:
                raise RuntimeError(f"probe launch failed: hipError {rc}")
        return step

    rows = []
    for name, step in (("the kernel as shipped", lambda i: r.enqueue(desc, wd, xd, bd, out)),
                       ("no output stores", variant(8)),
                       ("no fragment reads (tile loads + MFMAs + barriers + output)", variant(4)),
                       ("no tile loads, no output (fragment reads + MFMAs + barriers)", variant(9)),
                       ("MFMAs + barriers only (no tile loads, no fragment reads, no output)", variant(13)),
                       ("tile loads + barriers only (no MFMAs, no fragment reads, no output)", variant(14)),
                       ("barriers + output only (no tile loads, no MFMAs, no fragment reads)", variant(7)),
                       ("barriers only", variant(15))):
        stats = {}
        ms, mode = r.time_steps(step, 100, 10, 1, stats)
        rows.append({"variant": name, "us_per_launch": round(ms * 1e3, 2), "us_min": round(stats["ms_per_step_min"] * 1e3, 2),
                     "timing": mode})
    return {"gemm_ablation": rows, "shape": "X[512x2560] f16 . W[10240x2560]^T f16 + bias", "kernel": "gemm_nt_dl_kernel<160, 128, 3, 2>"}


def cpu_baseline(O, wbuf, x, bias, budget_s=1.5):
    """The oracle's reference path on the host cores, same inputs: median of >= 3 runs.  Returns
    (seconds, runs) for the whole path (dequantize W to f32, f32 GEMV, bias, cast) and the same for the
    path with the weights dequantized beforehand (f32 GEMV + bias on an f32 copy of W)."""
    N, K = 10240, 2560

    def median_time(call):
        times = []
        call()  # warm-up
        t_end = time.perf_counter() + budget_s
        while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 50):
            t0 = time.perf_counter()
            call()
            times.append(time.perf_counter() - t0)
        return float(np.median(times)), len(times)

    whole = median_time(lambda: O.matmul_ref(wbuf, O.Q8_0H, (N, K), x, O.F16, x.shape, bias, False, True, True))
    wf = O.q8_0_dequantize(wbuf, N * K, True).reshape(N, K)
    xf, bf = x.astype(np.float32), bias.astype(np.float32)
    amortised = median_time(lambda: O.matmul_ref(wf, O.F32, (N, K), xf, O.F32, xf.shape, bf, False, True, True))
    return whole, amortised


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-secondary", action="store_true", help="only the headline workload")
    ap.add_argument("--profile", action="store_true",
                    help="for runs under rocprofv3 --pmc: the timed launches only (no wall-clock cross-check of 40,000 launches, "
                         "no host-cost probe), so that the counter file holds a few thousand dispatches per kernel")
    ap.add_argument("--gemm-only", action="store_true",
                    help="run only the two C4 GEMM workloads (f16 and Q8_0H weights) and print their lines; for profiling")
    ap.add_argument("--c3-only", action="store_true",
                    help="run only the attention products of configs[2] and print their lines; for profiling")
    ap.add_argument("--attention-only", action="store_true",
                    help="run only the fused attention workloads (prefill, causal prefill, one decode step); for profiling")
    ap.add_argument("--q4k-only", action="store_true",
                    help="run only the Q4_K prefill workload (C5 at 256 rows) and print its line; for profiling")
    ap.add_argument("--read-calibration", action="store_true",
                    help="only time an empty launch and read-only passes over the rotated weight copies next to the GEMV")
    ap.add_argument("--issue-calibration", action="store_true",
                    help="time a wavefront's MFMAs, packed vector instructions and LDS fragment reads alone and mixed, and print the table")
    ap.add_argument("--gemm-ablation", action="store_true",
                    help="time the f16 tiled GEMM at the configs[3] shape next to timing-only builds of it with parts left out")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run 20 device-to-device copies of 256 MiB (reference dispatches for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; the Matmul path has no multi-GPU leg "
              f"(asked for --gpus {args.gpus}).", file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no host fallback.", file=sys.stderr)
        return 3
    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_per_dispatch": 256 << 20, "dispatches": 20}))
        return 0
    from oracle import oracle as O
    r = Runner()
    if args.issue_calibration:
        print(json.dumps(issue_calibration(r)))
        return 0

    if args.gemm_ablation:
        print(json.dumps(gemm_ablation(r)))
        return 0

    if args.read_calibration:
        print(json.dumps(read_calibration(r, O, min(args.steps, 2000), min(args.warmup, 100))))
        return 0
    if args.gemm_only:
        for g in (bench_f16_gemm(r, O, 100, 10), bench_q8_gemm(r, O, 100, 10), bench_f16_gemm(r, O, 50, 5, M=2048),
                  bench_f16_gemm(r, O, 50, 5, M=4096)):
            print(json.dumps({"workload": g["workload"], "tflops": round(g["tflops"], 1), "ms_per_step": g["ms"],
                              "frac_mfma_f16_peak": round(g["tflops"] / MFMA_F16_PEAK_TFLOPS, 4)}))
        return 0

    if args.c3_only:
        for g in c3_products(r, O):
            print(json.dumps(g))
        return 0

    if args.attention_only:
        for g in bench_attention(r, O):
            print(json.dumps(g))
        return 0

    if args.q4k_only:
        print(json.dumps(bench_q4k(r, O, (256,), 100)[0]))
        return 0

    head = bench_q8_gemv(r, O, 1, args.steps, args.warmup, wall_clock=not args.profile)
    wbuf, x, bias = head.pop("inputs")
    (cpu_s, cpu_n), (cpu_am_s, cpu_am_n) = cpu_baseline(O, wbuf, x, bias)

    # the metric's second half (f16 GEMM at the configs[3] shape) always runs: its roofline object is part of the line
    gemm_f16 = bench_f16_gemm(r, O, max(50, args.steps // 40), 10)

    secondary = []
    if not args.no_secondary:
        sec_steps = max(200, args.steps // 4)
        warm = bench_q8_gemv(r, O, 1, sec_steps, max(20, args.warmup // 4), copies=1)
        warm.pop("inputs"), warm.pop("stats")
        secondary.append({"workload": "C2 Q8_0 GEMV M=1, warm: one weight copy, resident in the Infinity Cache (not HBM)",
                          "value": round(warm["gbps"], 1), "unit": "GB/s", "ms_per_step": warm["ms"], "timing": warm["mode"]})
        for M in (4, 8):
            s = bench_q8_gemv(r, O, M, sec_steps, max(20, args.warmup // 4), seed=M)
            s.pop("inputs"), s.pop("stats")
            secondary.append({"workload": f"C2 Q8_0 GEMV M={M}", "value": round(s["gbps"], 1), "unit": "GB/s",
                              "ms_per_step": s["ms"], "timing": s["mode"], "frac_hbm_peak": round(s["gbps"] / HBM_PEAK_GBPS, 4)})
        gsteps = max(50, args.steps // 40)
        for g in (gemm_f16, bench_q8_gemm(r, O, gsteps, 10),
                  bench_q8_gemm(r, O, gsteps, 10, act=r.ffi.RT_ACT_GELU)):
            secondary.append({"workload": g["workload"], "value": round(g["tflops"], 1), "unit": "TFLOP/s",
                              "ms_per_step": g["ms"], "timing": g["mode"],
                              "frac_mfma_f16_peak": round(g["tflops"] / MFMA_F16_PEAK_TFLOPS, 4)})

        secondary += bench_elementwise(r, O)
        secondary += other_configs(r, O)

    line = {
        "metric": "q8_0_gemv_hbm_gbps_phi2_mlp",
        "value": round(head["gbps"], 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[1]: Q8_0 GEMV, Phi-2 decode MLP up-projection, x[1x2560] f16 . "
                        "Q8_0H W[10240x2560]^T + f16 bias, M=1",
            "weight_copies_rotated": head["copies"],
            "launch": head["mode"],
            "timed_regions": head["stats"]["regions"],
            "untimed_graph_replays_ahead_of_a_region": head["stats"]["cover_replays"],
            "ms_per_step_is": "median over the timed regions of `steps` launches each",
            "ms_per_step_min": head["stats"]["ms_per_step_min"],
            "ms_per_step_max": head["stats"]["ms_per_step_max"],
            "max_rel_err_vs_oracle": head["err"],
            # no HIP event involved: host clock around 2000 replays of a graph of one rotation, between two synchronisations
            "wall_clock_ms_per_step": head["stats"].get("wall_clock_ms_per_step"),
            "wall_clock_launches": head["stats"].get("wall_clock_launches"),
            "host_us_per_enqueue": None if args.profile else host_enqueue_cost(r, O),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(head["gbps"], 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(head["gbps"] / HBM_PEAK_GBPS, 4),
            "traffic": GEMV_TRAFFIC_BYTES,
            "algorithmic_bytes_per_launch": head["bytes"],
            "kernel": "gemv_q8h_rowdot_kernel<5, 1, 1, 4>",
        },
        "roofline_gemm": {
            "workload": gemm_f16["workload"],
            "bound": "mfma",
            "achieved": round(gemm_f16["tflops"], 1),
            "peak": MFMA_F16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(gemm_f16["tflops"] / MFMA_F16_PEAK_TFLOPS, 4),
            "traffic": GEMM_F16_TRAFFIC_BYTES,
            "algorithmic_flops_per_launch": gemm_f16["flops"],
            "algorithmic_bytes_per_launch": gemm_f16["bytes"],
            "ms_per_step": gemm_f16["ms"],
            "kernel": "gemm_nt_dl_kernel<160, 128, 3, 2>",
        },
        "cpu_baseline": {
            "value": round(head["bytes"] / cpu_s / 1e9, 3),
            "unit": "GB/s",
            "cores": O.lib().orc_num_threads(),
            "kind": "port",
            "sample": f"the same M=1 workload, full size, median of {cpu_n} runs "
                      f"({cpu_s * 1e3:.1f} ms each: dequantize W to f32, f32 GEMV, bias, cast)",
            # the same with the weights dequantized once beforehand (f32 GEMV + bias over a 105 MB f32 copy of W),
            # priced with the same algorithmic bytes
            "dequant_amortised": {"value": round(head["bytes"] / cpu_am_s / 1e9, 3), "unit": "GB/s",
                                  "ms": round(cpu_am_s * 1e3, 2), "runs": cpu_am_n},
        },
        "secondary": secondary,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
