#!/usr/bin/env python3
"""Headline benchmark: Q4_K decode GEMV over the Llama-3-8B projection set on one MI355X.

A step is one pass of the seven projections of one transformer layer
(q, k, v, o, gate, up, down) at M=1 with fp32 activations through ``qmm_matmul``.
Steps rotate over several distinct layers' weights so that no step finds its
weights in the 256 MB Infinity Cache.  The value is algorithmic bytes per step
(packed weight bytes + fp32 activations + fp32 outputs) over wall time, in GB/s.

Prints ONE JSON line.  ``roofline`` covers the dominant kernel (the Q4_K GEMV),
timed with HIP events on the launch stream; ``cpu_baseline`` is the CPU oracle
(a port of the reference CPU path, not the MAX binary) on a bounded sample of the
same workload; ``extra`` carries per-shape and secondary-config rates.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

# The launches are replayed from HIP graphs.  With the runtime's graph packet capture on (its default here) every
# kernel node costs about 0.5 us more than through the ordinary dispatch path, so it is switched off for the
# benchmark unless the caller has set it; it is a setting of the HIP runtime, read when it initialises.
os.environ.setdefault("DEBUG_CLR_GRAPH_PACKET_CAPTURE", "0")

import torch  # noqa: E402

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from mojo_amd import QuantizationConfig, QuantizationEncoding as QE  # noqa: E402
from mojo_amd import _lib, qmatmul, quantize, quantize_gptq  # noqa: E402

HBM_PEAK_GBS = 8000.0
BF16_PEAK_TFLOPS = 2500.0
PREFILL_KERNEL = "planes_prologue_kernel + gemm_planes_wide_kernel"

# (name, N, K) of the Llama-3-8B projections
PROJ = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
        ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)]


def alg_bytes(enc: QE, m: int, n: int, k: int) -> int:
    return n * enc.packed_row_bytes(k) + 4 * m * k + 4 * m * n


class Gemv:
    """One preallocated qmm_matmul call (no Python-side allocation when launched)."""

    def __init__(self, enc: QE, w: torch.Tensor, a: torch.Tensor, flags: int = 0):
        self.lib = _lib.load()
        self.enc, self.w, self.a, self.flags = enc, w, a, flags
        self.m, self.k = a.shape
        self.n = w.shape[0]
        self.out = torch.empty((self.m, self.n), dtype=torch.float32, device=a.device)
        dt = _lib.QMM_F32 if a.dtype == torch.float32 else _lib.QMM_BF16
        need = self.lib.qmm_matmul_workspace_bytes(enc.code, dt, self.m, self.n, self.k)
        self.ws = torch.empty((max(need, 1),), dtype=torch.uint8, device=a.device)
        self.need = need
        self.dt = dt
        self.ptrs = (C.c_void_p * 1)(w.data_ptr())

    def launch(self, stream_ptr: int) -> None:
        rc = self.lib.qmm_matmul(self.enc.code, None, C.c_void_p(self.a.data_ptr()), self.dt, self.m, self.k,
                                 self.ptrs, 1, self.n, C.c_void_p(self.out.data_ptr()),
                                 C.c_void_p(self.ws.data_ptr()), self.need, self.flags, C.c_void_p(stream_ptr))
        _lib.check(rc, "qmm_matmul")


class NormGemv(Gemv):
    """One preallocated qmm_matmul_rmsnorm call: RMS normalisation of the lhs rows, then the matmul."""

    def __init__(self, enc: QE, w: torch.Tensor, a: torch.Tensor, gamma: torch.Tensor, eps: float = 1e-5):
        super().__init__(enc, w, a)
        self.gamma, self.eps = gamma, eps
        self.need = self.lib.qmm_matmul_rmsnorm_workspace_bytes(enc.code, self.dt, self.m, self.n, self.k, 0)
        self.ws = torch.empty((max(self.need, 1),), dtype=torch.uint8, device=a.device)

    def launch(self, stream_ptr: int) -> None:
        rc = self.lib.qmm_matmul_rmsnorm(self.enc.code, None, C.c_void_p(self.a.data_ptr()), self.dt, C.c_void_p(self.gamma.data_ptr()),
                                         C.c_float(self.eps), self.m, self.k, self.ptrs, 1, self.n, C.c_void_p(self.out.data_ptr()),
                                         C.c_void_p(self.ws.data_ptr()), self.need, 0, C.c_void_p(stream_ptr))
        _lib.check(rc, "qmm_matmul_rmsnorm")


class GroupedGemv:
    """One preallocated qmm_matmul_grouped call: several weight matrices, one lhs."""

    def __init__(self, enc: QE, ws, a: torch.Tensor):
        self.lib = _lib.load()
        self.enc, self.ws_t, self.a = enc, list(ws), a
        self.m, self.k = a.shape
        self.outs = [torch.empty((self.m, w.shape[0]), dtype=torch.float32, device=a.device) for w in self.ws_t]
        self.dt = _lib.QMM_F32 if a.dtype == torch.float32 else _lib.QMM_BF16
        self.need = max(self.lib.qmm_matmul_workspace_bytes(enc.code, self.dt, self.m, w.shape[0], self.k) for w in self.ws_t)
        self.ws = torch.empty((max(self.need, 1),), dtype=torch.uint8, device=a.device)
        cnt = len(self.ws_t)
        self.cnt = cnt
        self.rhs_p = (C.c_void_p * cnt)(*[w.data_ptr() for w in self.ws_t])
        self.out_p = (C.c_void_p * cnt)(*[o.data_ptr() for o in self.outs])
        self.n_p = (C.c_int64 * cnt)(*[w.shape[0] for w in self.ws_t])

    def launch(self, stream_ptr: int) -> None:
        rc = self.lib.qmm_matmul_grouped(self.enc.code, C.c_void_p(self.a.data_ptr()), self.dt, self.m, self.k, self.cnt,
                                         self.rhs_p, self.n_p, self.out_p, C.c_void_p(self.ws.data_ptr()), self.need,
                                         C.c_void_p(stream_ptr))
        _lib.check(rc, "qmm_matmul_grouped")


class SwigluGemv:
    """One preallocated qmm_matmul_swiglu call: silu(lhs . gate^T) * (lhs . up^T)."""

    def __init__(self, enc: QE, gate: torch.Tensor, up: torch.Tensor, a: torch.Tensor):
        self.lib = _lib.load()
        self.enc, self.gate, self.up, self.a = enc, gate, up, a
        self.m, self.k = a.shape
        self.n = gate.shape[0]
        self.out = torch.empty((self.m, self.n), dtype=torch.float32, device=a.device)
        self.dt = _lib.QMM_F32 if a.dtype == torch.float32 else _lib.QMM_BF16
        self.need = self.lib.qmm_matmul_swiglu_workspace_bytes(enc.code, self.dt, self.m, self.n, self.k)
        self.ws = torch.empty((max(self.need, 1),), dtype=torch.uint8, device=a.device)

    def launch(self, stream_ptr: int) -> None:
        rc = self.lib.qmm_matmul_swiglu(self.enc.code, C.c_void_p(self.a.data_ptr()), self.dt, self.m, self.k,
                                        C.c_void_p(self.gate.data_ptr()), C.c_void_p(self.up.data_ptr()), self.n,
                                        C.c_void_p(self.out.data_ptr()), C.c_void_p(self.ws.data_ptr()), self.need,
                                        C.c_void_p(stream_ptr))
        _lib.check(rc, "qmm_matmul_swiglu")


class GptqMatmul:
    """One preallocated GPTQ qmm_matmul call on (qweight, scales, qzeros)."""

    def __init__(self, tensors, a: torch.Tensor, group: int = 128, g_idx=None):
        self.lib = _lib.load()
        self.t, self.a, self.g_idx = tensors, a, g_idx
        self.m, self.k = a.shape
        self.n = tensors[0].shape[1]
        self.out = torch.empty((self.m, self.n), dtype=torch.float32, device=a.device)
        self.dt = _lib.QMM_F32 if a.dtype == torch.float32 else _lib.QMM_BF16
        self.need = self.lib.qmm_matmul_workspace_bytes(QE.GPTQ.code, self.dt, self.m, self.n, self.k)
        self.ws = torch.empty((max(self.need, 1),), dtype=torch.uint8, device=a.device)
        self.cfg = _lib.GptqConfig(4, group, 0 if g_idx is None else 1, 1)  # g_idx given: an act-order checkpoint
        ptrs = [t.data_ptr() for t in tensors[:3]] + ([] if g_idx is None else [g_idx.data_ptr()])
        self.ptrs = (C.c_void_p * len(ptrs))(*ptrs)

    def launch(self, stream_ptr: int) -> None:
        rc = self.lib.qmm_matmul(QE.GPTQ.code, C.byref(self.cfg), C.c_void_p(self.a.data_ptr()), self.dt, self.m,
                                 self.k, self.ptrs, len(self.ptrs), self.n, C.c_void_p(self.out.data_ptr()),
                                 C.c_void_p(self.ws.data_ptr()), self.need, 0, C.c_void_p(stream_ptr))
        _lib.check(rc, "qmm_matmul")


class RepackedGemv:
    """One preallocated qmm_matmul_repacked call: the weight planes are made once, here, and every launch reuses them."""

    def __init__(self, enc: QE, rhs, a: torch.Tensor, group: int = 128):
        self.lib = _lib.load()
        self.enc, self.rhs, self.a = enc, tuple(rhs), a
        self.m, self.k = a.shape
        self.n = rhs[0].shape[1] if enc == QE.GPTQ else rhs[0].shape[0]
        self.cfg = _lib.GptqConfig(4, group, 0, 1) if enc == QE.GPTQ else None
        self.cfg_p = C.byref(self.cfg) if self.cfg else None
        self.ptrs = (C.c_void_p * len(self.rhs))(*[t.data_ptr() for t in self.rhs])
        size = self.lib.qmm_repack_bytes(enc.code, self.cfg_p, self.n, self.k)
        if size <= 0:
            raise ValueError("no weight planes for this encoding / shape")
        self.packed = torch.empty((size,), dtype=torch.uint8, device=a.device)
        self.repack(torch.cuda.current_stream().cuda_stream)
        self.out = torch.empty((self.m, self.n), dtype=torch.float32, device=a.device)
        self.dt = _lib.QMM_F32 if a.dtype == torch.float32 else _lib.QMM_BF16
        self.need = self.lib.qmm_matmul_repacked_workspace_bytes(enc.code, self.dt, self.m, self.n, self.k)
        self.ws = torch.empty((max(self.need, 1),), dtype=torch.uint8, device=a.device)

    def repack(self, stream_ptr: int) -> None:
        _lib.check(self.lib.qmm_repack(self.enc.code, self.cfg_p, self.ptrs, len(self.rhs), self.n, self.k,
                                       C.c_void_p(self.packed.data_ptr()), self.packed.numel(), C.c_void_p(stream_ptr)), "qmm_repack")

    def launch(self, stream_ptr: int) -> None:
        rc = self.lib.qmm_matmul_repacked(self.enc.code, self.cfg_p, C.c_void_p(self.a.data_ptr()), self.dt, self.m, self.k, self.ptrs,
                                          len(self.rhs), C.c_void_p(self.packed.data_ptr()), self.packed.numel(), self.n,
                                          C.c_void_p(self.out.data_ptr()), C.c_void_p(self.ws.data_ptr()), self.need, 0,
                                          C.c_void_p(stream_ptr))
        _lib.check(rc, "qmm_matmul_repacked")


class Repack:
    """The one-time conversion of a RepackedGemv as a launch of its own (for timing it)."""

    def __init__(self, call: RepackedGemv):
        self.call = call

    def launch(self, stream_ptr: int) -> None:
        self.call.repack(stream_ptr)


class ReadProbe:
    """qmm_read_probe over an existing tensor: the plain-read yardstick for the same bytes."""

    def __init__(self, t: torch.Tensor):
        self.lib = _lib.load()
        self.t = t
        self.nbytes = t.numel() * t.element_size() // 16 * 16

    def launch(self, stream_ptr: int) -> None:
        _lib.check(self.lib.qmm_read_probe(C.c_void_p(self.t.data_ptr()), self.nbytes, C.c_void_p(stream_ptr)),
                   "qmm_read_probe")


def make_weight(enc: QE, n: int, k: int, gen: torch.Generator) -> torch.Tensor:
    w = torch.randn((n, k), dtype=torch.float32, device="cuda:0", generator=gen) * 0.02
    return quantize(enc, w)


def capture(calls) -> torch.cuda.CUDAGraph:
    """Record a list of Gemv launches into one HIP graph on a side stream."""
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for c in calls:  # warm the kernels outside capture
            c.launch(s.cuda_stream)
        s.synchronize()
        with torch.cuda.graph(g, stream=s):
            sp = torch.cuda.current_stream().cuda_stream
            for c in calls:
                c.launch(sp)
    torch.cuda.current_stream().wait_stream(s)
    return g


def capture_forked(stages) -> torch.cuda.CUDAGraph:
    """Record stages of launches into one HIP graph; the launches of a stage are independent of each other and are
    recorded on streams of their own, so the graph holds them as parallel branches that join before the next stage."""
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    width = max(len(st) for st in stages)
    side = [torch.cuda.Stream() for _ in range(width - 1)]
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for st in stages:
            for c in st:
                c.launch(s.cuda_stream)
        s.synchronize()
        with torch.cuda.graph(g, stream=s):
            main = torch.cuda.current_stream()
            for st in stages:
                for x in side[:len(st) - 1]:
                    x.wait_stream(main)
                st[0].launch(main.cuda_stream)
                for c, x in zip(st[1:], side):
                    c.launch(x.cuda_stream)
                for x in side[:len(st) - 1]:
                    main.wait_stream(x)
    torch.cuda.current_stream().wait_stream(s)
    return g


MIN_TIMED_MS = 50.0   # a timed measurement covers at least this much device time, whatever --steps is
RAMP_MS = 30.0        # untimed replays before it, so that the clocks have left their idle state
HEADLINE_WARM_S = 1.0     # the headline warms up on a time basis (the reference's harness runs at least a second before
                          # it trusts a figure, stdlib/docs/bencher/BenchConfig.md: min_runtime_secs / max_runtime_secs)
HEADLINE_MIN_MS = 200.0   # device time covered by the headline's timed blocks
LAST_REPEATS = 0      # blocks of `steps` replays behind the last time_graphs() result


def time_graphs(graphs, steps: int, warmup: int, min_ms: float = MIN_TIMED_MS):
    """Seconds for exactly `steps` replays (graph i % len), HIP events on the launch stream.

    `warmup` untimed replays come first, then more until RAMP_MS of wall time has passed.  One block of exactly
    `steps` replays is timed between two events; blocks are repeated back to back (an event between them, one
    synchronisation at the end) until at least `min_ms` of device time is covered, and the MEDIAN block is
    returned, so that a short block (20 steps = 1 ms) reports the same rate as a long one.  Returns
    (device seconds of the median block, wall seconds per block); LAST_REPEATS holds the block count."""
    global LAST_REPEATS
    nxt = 0
    for _ in range(warmup):
        graphs[nxt % len(graphs)].replay()
        nxt += 1
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < RAMP_MS:
        for _ in range(max(1, min(steps, 64))):
            graphs[nxt % len(graphs)].replay()
            nxt += 1
        torch.cuda.synchronize()

    def run_blocks(count: int):
        nonlocal nxt
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(count + 1)]
        w0 = time.perf_counter()
        ev[0].record()
        for b in range(count):
            for _ in range(steps):
                graphs[nxt % len(graphs)].replay()
                nxt += 1
            ev[b + 1].record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - w0
        return [ev[b].elapsed_time(ev[b + 1]) for b in range(count)], wall

    first, _ = run_blocks(1)
    repeats = int(min(5000, max(3, -(-min_ms // max(first[0], 1e-3)))))
    times, wall = run_blocks(repeats)
    times.sort()
    LAST_REPEATS = repeats
    return times[len(times) // 2] * 1e-3, wall / repeats


class StepRunner:
    """The headline workload as graphs that hold whole steps, so that the host issues one launch per rotation of the
    layers instead of one per step: `full` holds one step of every layer (layers x 7 kernel nodes, each layer's own
    weights: a rotation reads 8 x 123 MB, so no step finds its weights in the 256 MB last-level cache), `rest` the first
    steps % layers layers.  A block is exactly `steps` steps: steps // layers replays of `full`, then `rest`."""

    def __init__(self, layer_calls, steps: int):
        self.layers = len(layer_calls)
        self.steps = steps
        self.full = capture([c for cs in layer_calls for c in cs])
        rem = steps % self.layers
        self.rest = capture([c for cs in layer_calls[:rem] for c in cs]) if rem else None
        self.host_launches_per_block = steps // self.layers + (1 if rem else 0)

    def block(self) -> None:
        for _ in range(self.steps // self.layers):
            self.full.replay()
        if self.rest is not None:
            self.rest.replay()

    def warm(self, steps: int, seconds: float) -> int:
        """At least `steps` untimed steps, then whole rotations until `seconds` of wall time have passed."""
        done, t0 = 0, time.perf_counter()
        while done < steps or time.perf_counter() - t0 < seconds:
            for _ in range(8):
                self.full.replay()
            done += 8 * self.layers
            torch.cuda.synchronize()
        return done

    def time(self, min_ms: float):
        """Blocks of exactly `steps` steps between HIP events on the launch stream, back to back, until `min_ms` of device
        time is covered.  Returns (sorted block times in ms, wall seconds per block)."""
        def run(count: int):
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(count + 1)]
            w0 = time.perf_counter()
            ev[0].record()
            for b in range(count):
                self.block()
                ev[b + 1].record()
            torch.cuda.synchronize()
            return [ev[b].elapsed_time(ev[b + 1]) for b in range(count)], time.perf_counter() - w0

        first, _ = run(1)
        repeats = int(min(5000, max(5, -(-min_ms // max(first[0], 1e-3)))))
        times, wall = run(repeats)
        return sorted(times), wall / repeats


def host_launch_cost_us(graph, count: int = 30) -> float:
    """Median host time of one graph launch call (the queue is empty when it is made)."""
    costs = []
    for _ in range(count):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        costs.append((time.perf_counter() - t0) * 1e6)
    torch.cuda.synchronize()
    costs.sort()
    return costs[len(costs) // 2]


class ClockSampler:
    """Samples the GPU's current shader clock (MHz) from the amdgpu driver's sysfs files while a region runs.
    `mhz` is the median sample, or None where the files are absent or unreadable."""

    def __init__(self, period_s: float = 0.005):
        import glob
        import threading

        self.paths = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/freq1_input"))
        self.dpm = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.period, self.samples, self.stop = period_s, [], threading.Event()
        self.thread = threading.Thread(target=self._run, daemon=True)

    def _read(self):
        best = None
        for p in self.paths:
            try:
                v = int(open(p).read().strip()) / 1e6
                best = v if best is None else max(best, v)  # (several cards: the busy one has the highest clock)
            except (OSError, ValueError):
                pass
        if best is None:
            for p in self.dpm:
                try:
                    for line in open(p).read().splitlines():
                        if line.rstrip().endswith("*"):
                            v = float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
                            best = v if best is None else max(best, v)
                except (OSError, ValueError, IndexError):
                    pass
        return best

    def _run(self):
        while not self.stop.is_set():
            v = self._read()
            if v:
                self.samples.append(v)
            time.sleep(self.period)

    def __enter__(self):
        self.thread.start()
        return self

    def __exit__(self, *exc):
        self.stop.set()
        self.thread.join()

    @property
    def mhz(self):
        if not self.samples:
            return None
        s = sorted(self.samples)
        return s[len(s) // 2]


def host_cpu():
    """(model name, physical cores visible) from /proc/cpuinfo; the pair (physical id, core id) names a core
    (the count the reference's num_physical_cores reports, stdlib/src/sys/info.mojo:789-796)."""
    model, cores, phys, core = "unknown", set(), None, None
    try:
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name":
                model = val
            elif key == "physical id":
                phys = val
            elif key == "core id":
                core = val
            elif not key and phys is not None:
                cores.add((phys, core))
                phys = core = None
        if phys is not None:
            cores.add((phys, core))
    except OSError:
        pass
    return model, len(cores) or (os.cpu_count() or 1)


def cpu_baseline(layer_w, m: int, budget_s: float = 10.0):
    """Port of the reference CPU path (the oracle's source) on one layer's seven projections, OpenMP over N.

    Three variants are timed and the fastest is reported (all named in `sample`): the portable exactness-grade build
    that the tests check against, a build of the same source for this host (-O3 -march=native, contraction on, made
    here with `make -C oracle native`), and the library's hand-vectorised AVX2 + FMA kernel with the unpack fused into
    the dot.  Threads: the physical cores, capped at this job's share of the host."""
    import subprocess

    import numpy as np

    import oracle as O

    model, phys = host_cpu()
    share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or 16  # the job's share of the host's cores
    threads = max(1, min(phys, share, O.num_threads() if O.num_threads() > 0 else share))
    port = lambda lib: (lambda a, w: lib.matmul_f32(O.Q4_K, a, w))  # noqa: E731
    builds = [("portable build (-march=x86-64-v3, contraction off: the one the tests check against)", O, port(O))]
    try:
        subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "native"], check=True, capture_output=True, timeout=120)
        nat = O.native()
        builds.append(("-O3 -march=native build of the same source", nat, port(nat)))
    except Exception as exc:  # no compiler, or a CPU the build does not suit: the portable library still times the port
        builds[0] = (builds[0][0] + f"; native build unavailable: {type(exc).__name__}",) + builds[0][1:]
    rng = np.random.Generator(np.random.PCG64(3))
    host = [(w.cpu().numpy(), n, k) for (w, (_, n, k)) in zip(layer_w, PROJ)]
    acts = {k: rng.standard_normal((m, k), dtype=np.float32) for k in (4096, 14336)}
    # the hand-vectorised (AVX2 + FMA) fused unpack-and-dot of the same library, where the host has AVX2
    if O.baseline_matmul_q4_k(acts[4096][:1], host[0][0][:8]) is not None:
        builds.append(("hand-vectorised AVX2 + FMA kernel (unpack fused into the dot)", O, O.baseline_matmul_q4_k))
    nbytes = sum(alg_bytes(QE.Q4_K, m, n, k) for _, n, k in PROJ)
    results = []
    for what, lib, fn in builds:  # each variant gets its share of the budget; the fastest one is the baseline
        lib.set_num_threads(threads)
        for w, n, k in host:  # warm-up pass
            fn(acts[k], w)
        passes, t0 = 0, O.now()
        while True:
            for w, n, k in host:
                fn(acts[k], w)
            passes += 1
            el = O.now() - t0
            if el > budget_s / len(builds) or passes >= 5000:
                break
        results.append((nbytes * passes / el / 1e9, passes, el, what))
    best = max(results)
    others = "; ".join(f"{r[3]}: {r[0]:.1f} GB/s" for r in results if r is not best)
    return {"value": round(best[0], 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{best[1]} passes of one layer's 7 Q4_K projections at M={m} ({nbytes} B each), "
                      f"{best[2]:.1f} s, OpenMP over N on {threads} threads; host: {model}, {phys} physical cores, "
                      f"{os.cpu_count()} logical cpus; timed: {best[3]}" + (f" (also timed: {others})" if others else "")}


def measured_traffic(key: str):
    """HBM bytes per launch from the committed PMC summary (profiles/hbm_traffic.json), or None.  The entry names the kernel
    sources it was measured on (a hash): a figure taken on other sources than the tree's is not reported."""
    import hashlib

    files = {"decode_m1": ("gemv_q4k_lanes.hip", "lds_stream.h"), "prefill_q4_k": ("gemm_planes.hip", "gemm_tile.h", "gemm_lhs.h")}
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            entry = json.load(f)[key]
        h = hashlib.sha256()
        for name in files[key]:
            with open(os.path.join(ROOT, "mojo_amd", "csrc", name), "rb") as src:
                h.update(src.read())
        if entry.get("source_sha256_16") != h.hexdigest()[:16]:
            return None
        return entry["traffic_bytes_per_launch"]
    except (OSError, KeyError, ValueError):
        return None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=8, help="distinct layers of weights to rotate over")
    ap.add_argument("--m", type=int, default=1, help="lhs rows of the headline workload (1 or 4)")
    ap.add_argument("--workload", choices=("decode", "prefill", "gptq_prefill", "q6k_prefill", "q5k_prefill", "q40_prefill", "calib", "mfma_probe", "sweep", "ladder", "ladder_other"),
                    default="decode",
                    help="decode: the headline Q4_K GEMV set; prefill / gptq_prefill / q6k_prefill / q5k_prefill / q40_prefill: the M=2048 "
                         "GEMM of the same model's gate projection (second target, matrix-core roofline); calib: a plain "
                         "read and a plain copy of 256 MiB, the yardsticks for the FETCH_SIZE / WRITE_SIZE counters; mfma_probe: the "
                         "matrix-core rate of a register-resident loop by operand data; sweep: Q4_K decode and prefill over shapes "
                         "the dispatch was not tuned on; ladder: every encoding over 1 .. 256 lhs rows of both types on two projection shapes")
    ap.add_argument("--repacked", action="store_true", help="prefill workloads: weight planes made once (qmm_repack), outside the timed steps")
    ap.add_argument("--min-ms", type=float, default=HEADLINE_MIN_MS,
                    help="device time the headline's timed blocks cover at least (profiler runs pass a small value to keep their traces short)")
    ap.add_argument("--warm-seconds", type=float, default=HEADLINE_WARM_S,
                    help="decode: least wall time of the headline's warm-up (profiling runs shorten it to keep their traces small)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip per-shape and secondary-config timings")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill GEMM leg (roofline_prefill)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this path runs on a single MI355X and --gpus {args.gpus} is not "
              "supported (the path would shard by output columns N across GPUs; that is not built).", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(3)
    if args.workload == "calib":
        return calib_main()
    if args.workload == "mfma_probe":
        return probe_main()
    if args.workload == "sweep":
        return sweep_main(gen)
    if args.workload == "ladder":
        return ladder_main(gen)
    if args.workload == "ladder_other":
        return ladder_main(gen, LADDER_OTHER_SHAPES, LADDER_OTHER_ROWS)
    if args.workload != "decode":
        return prefill_main(args, gen)
    m = args.m
    acts = {k: torch.randn((m, k), dtype=torch.float32, device="cuda:0", generator=gen) for k in (4096, 14336)}
    layers = []
    for _ in range(args.layers):
        layers.append([make_weight(QE.Q4_K, n, k, gen) for _, n, k in PROJ])
    calls = [[Gemv(QE.Q4_K, w, acts[k]) for w, (_, n, k) in zip(lw, PROJ)] for lw in layers]
    step_bytes = sum(alg_bytes(QE.Q4_K, m, n, k) for _, n, k in PROJ)

    # The headline: graphs that hold whole steps (one host launch per rotation of the layers), a warm-up of at least a
    # second, nothing else running in this process while the blocks are timed.
    runner = StepRunner(calls, args.steps)
    warm_steps = runner.warm(args.warmup, args.warm_seconds)
    times, wall_s = runner.time(args.min_ms)
    repeats = len(times)
    dev_s = times[repeats // 2] * 1e-3
    ms_per_step = dev_s * 1e3 / args.steps
    value = step_bytes * args.steps / dev_s / 1e9
    launches = args.steps * len(PROJ)
    avg_launch_us = dev_s * 1e6 / launches
    avg_launch_bytes = step_bytes / len(PROJ)
    achieved = avg_launch_bytes / (avg_launch_us * 1e-6) / 1e9
    # the shader clock under this load, sampled over replays of their own after the timed blocks
    with ClockSampler() as clk:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.15:
            runner.full.replay()
            torch.cuda.synchronize()

    cu, khz = C.c_int32(0), C.c_int32(0)
    _lib.load().qmm_device_info(C.byref(cu), C.byref(khz))

    us = lambda ms: round(ms * 1e3 / args.steps, 3)  # noqa: E731
    extra = {"wall_ms_per_step": round(wall_s * 1e3 / args.steps, 5), "avg_launch_us": round(avg_launch_us, 3),
             "compute_units": cu.value, "clock_mhz": khz.value / 1000.0, "clock_mhz_during_decode": clk.mhz,
             "headline_blocks_us_per_step": {"min": us(times[0]), "median": us(times[repeats // 2]), "max": us(times[-1]),
                                             "p10": us(times[repeats // 10]), "p90": us(times[repeats * 9 // 10])},
             "headline_warmup_steps": warm_steps,
             "host_launches_per_block": runner.host_launches_per_block,
             "host_us_per_graph_launch": {f"{args.layers * len(PROJ)}_kernel_nodes": round(host_launch_cost_us(runner.full), 1)}}
    if not args.no_extra:
        # The same steps issued as one 7-node graph per step (a host launch every step): where this is slower than the
        # headline, the host is the limiter, not the GPU.
        small = [capture(c) for c in calls]
        extra["host_us_per_graph_launch"]["7_kernel_nodes"] = round(host_launch_cost_us(small[0]), 1)
        d7, w7 = time_graphs(small, args.steps, args.warmup)
        extra["one_graph_launch_per_step"] = {"us_per_step": round(d7 * 1e6 / args.steps, 3), "wall_us_per_step": round(w7 * 1e6 / args.steps, 3),
                                              "GB/s": round(step_bytes * args.steps / d7 / 1e9, 1)}
        with ClockSampler():
            d7s, _ = time_graphs(small, args.steps, args.warmup)
        extra["one_graph_launch_per_step"]["us_per_step_with_clock_sampler_thread"] = round(d7s * 1e6 / args.steps, 3)
        del small
    roofline_prefill = None if args.no_prefill else prefill_roofline(gen, cu.value, khz.value / 1000.0)
    if roofline_prefill is not None:
        roofline_prefill["mfma_probe"] = mfma_probe()
    if not args.no_extra:
        extra.update(extra_timings(layers, acts, gen))
        # the headline once more, after everything else: the same graphs, a short warm-up
        runner.warm(args.warmup, 0.2)
        t2, _ = runner.time(args.min_ms / 2)
        extra["headline_remeasured_at_end"] = {"us_per_step": us(t2[len(t2) // 2]), "min": us(t2[0]), "max": us(t2[-1]),
                                               "GB/s": round(step_bytes * args.steps / (t2[len(t2) // 2] * 1e-3) / 1e9, 1)}

    traffic = measured_traffic("decode_m1") if m == 1 and args.layers == 8 else None
    result = {
        "metric": "Q4_K decode GEMV HBM GB/s",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "repeats": repeats,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"Q4_K decode GEMV, Llama-3-8B projection set (q,k,v,o,gate,up,down), M={m}, fp32 "
                        f"activations, fp32 out; weights 0.02*N(0,1) quantised to Q4_K on the GPU, activations "
                        f"N(0,1); {args.layers} distinct layers rotated (cold cache); one step = one layer "
                        f"= 7 qmm_matmul launches, {step_bytes} algorithmic bytes",
            "m": m, "layers": args.layers, "bytes_per_step": step_bytes,
            "inputs": "torch.Generator(cuda:0) seed 3: weights randn * 0.02 packed by qmm_quantize (bit-exact with the "
                      "oracle's packer), activations randn",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "kernel": "gemv_q4_k_lanes_plain_kernel",
            "bytes_per_launch": avg_launch_bytes,
            "launch_us": round(avg_launch_us, 3),
        },
        "roofline_prefill": roofline_prefill,
        "extra": extra,
    }
    extra["timing"] = (f"ms_per_step is the median of {repeats} timed blocks of exactly {args.steps} steps each, run back to back "
                       f"after {warm_steps} warm-up steps (at least {args.warmup}, and at least {args.warm_seconds:.2f} s); a block is "
                       f"{runner.host_launches_per_block} graph launches (a graph holds one step of each of the {args.layers} layers)")
    extra["DEBUG_CLR_GRAPH_PACKET_CAPTURE"] = os.environ.get("DEBUG_CLR_GRAPH_PACKET_CAPTURE")
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(layers[0], m)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))
    return 0


def prefill_roofline(gen, cus: int, nominal_mhz: float):
    """Second half of the metric: the Q4_K prefill GEMM (bf16 lhs [2048, 4096] x Q4_K [14336, 4096], fp32 out)
    against the dense fp16 / bf16 matrix-core peak, and against that peak scaled to the shader clock the driver
    reports while the kernel runs (compute units x 4 SIMDs x 1024 flop per clock x clock)."""
    mm, n, k = 2048, 14336, 4096
    ab = torch.randn((mm, k), dtype=torch.float32, device="cuda:0", generator=gen).to(torch.bfloat16)
    call = Gemv(QE.Q4_K, make_weight(QE.Q4_K, n, k, gen), ab)
    g = capture([call])
    dev_s, _ = time_graphs([g], 10, 3, min_ms=150.0)
    with ClockSampler() as clk:  # the clock under this kernel, over replays of their own
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.15:
            g.replay()
            torch.cuda.synchronize()
    us = dev_s * 1e6 / 10
    flops = 2.0 * mm * n * k
    tf = flops / us / 1e6
    mhz = clk.mhz
    peak_at_clock = cus * 4 * 1024 * mhz * 1e6 / 1e12 if mhz else None
    # the same product with the weight planes made once (qmm_repack) instead of in every call
    kept = RepackedGemv(QE.Q4_K, (call.w,), ab)
    dev_s, _ = time_graphs([capture([kept])], 10, 3, min_ms=150.0)
    kept_us = dev_s * 1e6 / 10
    dev_s, _ = time_graphs([capture([Repack(kept)])], 10, 3, min_ms=50.0)
    repacked = {"launch_us": round(kept_us, 2), "achieved": round(flops / kept_us / 1e6, 2), "frac": round(flops / kept_us / 1e6 / BF16_PEAK_TFLOPS, 4),
                "kernel": "planes_prologue_kernel (lhs rows only) + gemm_planes_wide_kernel", "repack_us_once": round(dev_s * 1e6 / 10, 2),
                "packed_bytes": kept.packed.numel(),
                "note": "qmm_matmul_repacked on planes made once by qmm_repack, as a host that converts at model load would call it"}
    return {"bound": "mfma", "achieved": round(tf, 2), "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tf / BF16_PEAK_TFLOPS, 4), "traffic": measured_traffic("prefill_q4_k"), "kernel": PREFILL_KERNEL, "flops_per_launch": flops,
            "launch_us": round(us, 2), "clock_mhz_during_kernel": mhz,
            "peak_at_measured_clock": round(peak_at_clock, 1) if peak_at_clock else None,
            "frac_at_measured_clock": round(tf / peak_at_clock, 4) if peak_at_clock else None,
            "workload": f"Q4_K prefill GEMM, bf16 lhs [{mm}, {k}] x Q4_K weights [{n}, {k}], fp32 out; launch_us covers the "
                        "preparation kernel (lhs narrowing, weights to fp16 integer planes) and the GEMM",
            "repacked": repacked}


def mfma_probe(seconds: float = 0.12):
    """The matrix-core rate that a register-resident loop of v_mfma_f32_32x32x16_f16 sustains on this part (qmm_mfma_probe: no
    memory traffic, 8 wavefronts per compute unit), for zeros, for dense random data on both sides, and for random values
    against integers 0..945 (what the plane GEMMs multiply); each after `seconds` of untimed launches and over `seconds` of
    timed ones, with the shader clock sampled over launches of its own."""
    lib = _lib.load()
    cu = C.c_int32(0)
    lib.qmm_device_info(C.byref(cu), None)
    out = torch.empty((cu.value * 512,), dtype=torch.float32, device="cuda:0")
    s = torch.cuda.current_stream().cuda_stream
    iters, res = 2000, {}
    for kind, name in ((0, "zeros"), (2, "random_x_random"), (3, "random_x_integers_0_945"), (4, "zeros_16x16x32"), (5, "random_x_random_16x16x32"),
                       (6, "random_x_random_bf16")):
        flops = C.c_int64(0)

        def launch():
            _lib.check(lib.qmm_mfma_probe(C.c_void_p(out.data_ptr()), out.numel() * 4, kind, iters, C.byref(flops), C.c_void_p(s)), "qmm_mfma_probe")

        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(8):
                launch()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        count = 0
        e0.record()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(8):
                launch()
            count += 8
        e1.record()
        torch.cuda.synchronize()
        tf = flops.value * count / (e0.elapsed_time(e1) * 1e-3) / 1e12
        with ClockSampler() as clk:
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 0.06:
                for _ in range(8):
                    launch()
                torch.cuda.synchronize()
        res[name] = {"TFLOP/s": round(tf, 1), "frac_of_2500": round(tf / BF16_PEAK_TFLOPS, 4), "clock_mhz": clk.mhz}
    return res


def probe_main() -> int:
    print(json.dumps({"metric": "register-resident v_mfma_f32_32x32x16_f16 loop, TFLOP/s by operand data", "unit": "TFLOP/s",
                      "peak": BF16_PEAK_TFLOPS, "mfma_probe": mfma_probe(0.3)}))
    return 0


SWEEP_SHAPES = [(4096, 11008), (11008, 4096), (32000, 4096), (5120, 5120), (3584, 18944)]  # (N, K): none of them tuned for


def sweep_main(gen) -> int:
    """Q4_K over shapes the dispatch thresholds were not fitted to: lhs rows 1 / 4 / 16 / 64 (fp32) as a fraction of the plain read of the
    same weight bytes (cold: copies rotated beyond the 256 MB cache), prefill rows 512 / 2048 (bf16 lhs) as a fraction of the
    2.5 PFLOP/s peak.  One JSON line; a cliff in the dispatch shows as a fraction far below its neighbours'."""
    out = {}
    for n, k in SWEEP_SHAPES:
        w0 = make_weight(QE.Q4_K, n, k, gen)
        copies = max(2, (320 << 20) // w0.numel() + 1)
        ws = [w0] + [w0.clone() for _ in range(copies - 1)]
        dev_s, _ = time_graphs([capture([ReadProbe(w) for w in ws])], 20, 3)
        read_us = dev_s * 1e6 / (20 * copies)
        row = {"plain_read_us": round(read_us, 2), "plain_read_GB/s": round(w0.numel() / read_us / 1e3, 1)}
        for m in (1, 4, 16, 64):
            a = torch.randn((m, k), dtype=torch.float32, device="cuda:0", generator=gen)
            dev_s, _ = time_graphs([capture([Gemv(QE.Q4_K, w, a) for w in ws])], 20, 3)
            us = dev_s * 1e6 / (20 * copies)
            row[f"m{m}"] = {"us": round(us, 2), "GB/s": round(alg_bytes(QE.Q4_K, m, n, k) / us / 1e3, 1), "frac_of_plain_read": round(read_us / us, 3)}
        del ws
        for m in (512, 2048):
            ab = torch.randn((m, k), dtype=torch.float32, device="cuda:0", generator=gen).to(torch.bfloat16)
            dev_s, _ = time_graphs([capture([Gemv(QE.Q4_K, w0, ab)])], 10, 2)
            us = dev_s * 1e6 / 10
            tf = 2.0 * m * n * k / us / 1e6
            row[f"m{m}"] = {"us": round(us, 1), "TFLOP/s": round(tf, 1), "frac_of_2500": round(tf / BF16_PEAK_TFLOPS, 4)}
        out[f"{n}x{k}"] = row
        del w0
    print(json.dumps({"metric": "Q4_K over untuned shapes: decode as a fraction of the plain read, prefill of the matrix-core peak",
                      "encoding": "Q4_K", "sweep": out}))
    return 0


LADDER_ROWS = (1, 4, 8, 16, 17, 32, 64, 65, 128, 256)
LADDER_SHAPES = ((4096, 4096), (14336, 4096), (4096, 14336))
# projection shapes of other models (Llama-2-7B, 13B-like, 70B), a vocabulary of 32000, a K that is no multiple of 512 or 2048
LADDER_OTHER_SHAPES = ((11008, 4096), (4096, 11008), (5120, 5120), (8192, 8192), (32000, 4096), (28672, 8192), (8192, 28672))
LADDER_OTHER_ROWS = (1, 2, 4, 8, 16, 32, 64, 128, 256)


def ladder_main(gen, shapes=LADDER_SHAPES, rows=LADDER_ROWS) -> int:
    """Microseconds per qmm_matmul call for every encoding over 1 .. 256 lhs rows, fp32 and bf16, on the q / o, the gate / up and
    the down shape (24 calls per graph on one weight tensor, so the weights come from the last-level cache: the figures compare
    row counts and lhs types of one shape, not shapes).  One JSON line; a step between neighbouring row counts that is
    larger than the rows explain is a threshold of the dispatch in the wrong place.  ladder_other: the same over shapes
    that no threshold was fitted on."""
    out = {}
    for enc in (QE.Q4_K, QE.Q5_K, QE.Q6_K, QE.Q4_0, QE.GPTQ):
        for n, k in shapes:
            if enc == QE.GPTQ:
                w = quantize_gptq(torch.randn((n, k), dtype=torch.float32, device="cuda:0", generator=gen) * 0.02)
            else:
                w = make_weight(enc, n, k, gen)
            for dt, name in ((torch.float32, "f32"), (torch.bfloat16, "bf16")):
                row = {}
                for m in rows:
                    a = torch.randn((m, k), dtype=torch.float32, device="cuda:0", generator=gen).to(dt)
                    # (24 calls per graph: a graph launch costs the host about 20 us plus 3 us per kernel node, so six calls
                    # per graph would put a floor of 6 us under every figure)
                    calls = [GptqMatmul(w, a) if enc == QE.GPTQ else Gemv(enc, w, a) for _ in range(24)]
                    dev_s, _ = time_graphs([capture(calls)], 10, 2)
                    row[f"m{m}"] = round(dev_s * 1e6 / (10 * len(calls)), 1)
                    del calls
                out[f"{enc.name} {n}x{k} {name}"] = row
            del w
    print(json.dumps({"metric": "microseconds per call over lhs rows 1 .. 256, every encoding, both lhs types (warm weights)", "ladder": out}))
    return 0


def calib_main() -> int:
    """Known-size kernels for scaling the HBM counters: qmm_read_probe reads 256 MiB, a torch copy reads
    and writes 256 MiB.  Each runs three times; buffers are larger than every cache."""
    nbytes = 256 << 20
    src = torch.empty((nbytes,), dtype=torch.uint8, device="cuda:0").random_(0, 255)
    dst = torch.empty_like(src)
    probe = ReadProbe(src)
    s = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        probe.launch(s)
        dst.copy_(src)
    torch.cuda.synchronize()
    print(json.dumps({"calibration": {"read_probe_bytes": probe.nbytes, "copy_bytes_each_way": nbytes}}))
    return 0


def prefill_main(args, gen) -> int:
    """Second target: bf16 lhs [2048, 4096] x 4-bit weights [14336, 4096], one launch per step."""
    mm, n, k = 2048, 14336, 4096
    steps, warmup = min(args.steps, 50), min(args.warmup, 5)
    ab = torch.randn((mm, k), dtype=torch.float32, device="cuda:0", generator=gen).to(torch.bfloat16)
    if args.workload == "prefill":
        call, name, kern = Gemv(QE.Q4_K, make_weight(QE.Q4_K, n, k, gen), ab), "Q4_K", PREFILL_KERNEL
    elif args.workload == "q6k_prefill":
        call, name, kern = Gemv(QE.Q6_K, make_weight(QE.Q6_K, n, k, gen), ab), "Q6_K", "planes_prologue_kernel + gemm_planes2_kernel"
    elif args.workload == "q40_prefill":
        call, name, kern = Gemv(QE.Q4_0, make_weight(QE.Q4_0, n, k, gen), ab), "Q4_0", "q4_0_planes_prologue_kernel + gemm_q4_0_planes_kernel"
    elif args.workload == "q5k_prefill":
        call, name, kern = Gemv(QE.Q5_K, make_weight(QE.Q5_K, n, k, gen), ab), "Q5_K", "planes_prologue_kernel + gemm_planes_wide_kernel"
    else:
        wg = quantize_gptq(torch.randn((n, k), dtype=torch.float32, device="cuda:0", generator=gen) * 0.02)
        call, name, kern = GptqMatmul(wg, ab), "GPTQ g128", "gptq_planes_prologue_kernel + gemm_planes_wide_kernel"
    step_text = "one preparation launch (lhs narrowing, weights to fp16 integer planes) + one GEMM launch"
    if args.repacked:
        rhs = tuple(call.t[:3]) if args.workload == "gptq_prefill" else (call.w,)
        call = RepackedGemv(call.enc if hasattr(call, "enc") else QE.GPTQ, rhs, ab)
        kern = "planes_prologue_kernel (lhs rows only) + " + kern.split(" + ")[1]
        step_text = "one preparation launch (lhs narrowing) + one GEMM launch over weight planes made once by qmm_repack"
    g = capture([call])
    dev_s, wall_s = time_graphs([g], steps, warmup)
    us = dev_s * 1e6 / steps
    flops = 2.0 * mm * n * k
    tf = flops / us / 1e6
    print(json.dumps({
        "metric": f"{name} prefill GEMM TFLOP/s", "value": round(tf, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(us / 1e3, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 products, f32 sums", "data": "synthetic",
        "config": {"workload": f"{name} prefill GEMM, bf16 lhs [{mm}, {k}] x weights [{n}, {k}], fp32 out; one step = "
                               f"{step_text}", "m": mm, "n": n, "k": k},
        "roofline": {"bound": "mfma", "achieved": round(tf, 2), "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tf / BF16_PEAK_TFLOPS, 4), "traffic": None, "kernel": kern,
                     "flops_per_launch": flops, "launch_us": round(us, 2),
                     "note": "launch_us includes the preparation kernel (lhs narrowing" + ("" if args.repacked else ", weight planes") + ")"},
        "cpu_baseline": None,
    }))
    return 0


def extra_timings(layers, acts, gen):
    """Per-shape cold-cache rates for the headline set, M=4, and the other configs."""
    out = {}
    m = acts[4096].shape[0]
    # per projection shape, rotating over the layers' copies of that shape
    per_shape = {}
    for idx, (name, n, k) in enumerate(PROJ):
        if name in ("v", "up"):
            continue
        ws = [lw[idx] for lw in layers]
        if name in ("q", "k"):  # the same-shape sibling too
            ws += [lw[idx + (3 if name == "q" else 1)] for lw in layers]
        while sum(w.numel() for w in ws) < 320 << 20:  # copies, until a rotation is larger than the 256 MB cache
            ws += [w.clone() for w in ws[:len(layers)]]
        cs = [Gemv(QE.Q4_K, w, acts[k]) for w in ws]
        g = capture(cs)
        dev_s, _ = time_graphs([g], 50, 5)
        us = dev_s * 1e6 / (50 * len(cs))
        b = alg_bytes(QE.Q4_K, m, n, k)
        per_shape[f"{name}_{n}x{k}"] = {"us": round(us, 3), "GB/s": round(b / us / 1e3, 1)}
    out["q4_k_per_shape"] = per_shape
    # the floor under every launch: a kernel that reads 4 KB and does nothing else, 56 of them in a replayed graph
    tiny = torch.zeros((4096,), dtype=torch.uint8, device="cuda:0")
    dev_s, _ = time_graphs([capture([ReadProbe(tiny) for _ in range(56)])], 50, 5)
    out["launch_floor_us_per_kernel_node"] = round(dev_s * 1e6 / (50 * 56), 3)
    # warm cache, labelled as such: one layer (123 MB, inside the 256 MB last-level cache) replayed by itself
    g = capture([Gemv(QE.Q4_K, w, acts[k]) for w, (_, n, k) in zip(layers[0], PROJ)])
    dev_s, _ = time_graphs([g], 100, 10)
    sbw = sum(alg_bytes(QE.Q4_K, m, n, k) for _, n, k in PROJ)
    out["q4_k_warm_cache_one_layer"] = {"us_per_step": round(dev_s * 1e6 / 100, 2), "GB/s": round(sbw * 100 / dev_s / 1e9, 1)}
    # the same seven weight tensors per layer, only read (no arithmetic): what the memory system gives
    graphs = [capture([ReadProbe(w) for w in lw]) for lw in layers]
    dev_s, _ = time_graphs(graphs, 100, 10)
    wbytes = sum(n * QE.Q4_K.packed_row_bytes(k) for _, n, k in PROJ)
    out["plain_read_same_set"] = {"us_per_step": round(dev_s * 1e6 / 100, 2), "GB/s": round(wbytes * 100 / dev_s / 1e9, 1)}
    # the same step with the projections that share their lhs in one launch each: q|k|v, o, gate|up, down
    if m == 1:
        graphs = [capture([GroupedGemv(QE.Q4_K, lw[0:3], acts[4096]), Gemv(QE.Q4_K, lw[3], acts[4096]),
                           GroupedGemv(QE.Q4_K, lw[4:6], acts[4096]), Gemv(QE.Q4_K, lw[6], acts[14336])]) for lw in layers]
        dev_s, _ = time_graphs(graphs, 100, 10)
        sb = sum(alg_bytes(QE.Q4_K, m, n, k) for _, n, k in PROJ)
        out["q4_k_m1_grouped_4_launches"] = {"us_per_step": round(dev_s * 1e6 / 100, 2), "GB/s": round(sb * 100 / dev_s / 1e9, 1)}
        # ... and with the gate | up launch also applying silu(gate) * up (one output of 14336 instead of two)
        graphs = [capture([GroupedGemv(QE.Q4_K, lw[0:3], acts[4096]), Gemv(QE.Q4_K, lw[3], acts[4096]),
                           SwigluGemv(QE.Q4_K, lw[4], lw[5], acts[4096]), Gemv(QE.Q4_K, lw[6], acts[14336])]) for lw in layers]
        dev_s, _ = time_graphs(graphs, 100, 10)
        out["q4_k_m1_grouped_gated_4_launches"] = {"us_per_step": round(dev_s * 1e6 / 100, 2),
                                                   "GB/s": round((sb - 4 * 14336) * 100 / dev_s / 1e9, 1)}
        # seven qmm_matmul calls per step, with the ones that share their lhs (q, k, v and gate, up) as parallel
        # branches of the graph: stages (q | k | v), o, (gate | up), down
        cs = [[Gemv(QE.Q4_K, w, acts[k]) for w, (_, n, k) in zip(lw, PROJ)] for lw in layers]
        g = capture_forked([st for c in cs for st in (c[0:3], c[3:4], c[4:6], c[6:7])])
        dev_s, _ = time_graphs([g], 20, 3)
        out["q4_k_m1_forked_branches_7_launches"] = {"us_per_step": round(dev_s * 1e6 / (20 * len(layers)), 2),
                                                     "GB/s": round(sb * 20 * len(layers) / dev_s / 1e9, 1)}
        del g, cs
    # the optional integer-activation treatment (lhs -> Q8_K in the kernel, integer sub-block dots), M = 1 and 4
    for mm in (1, 4):
        a8 = {kk: torch.randn((mm, kk), dtype=torch.float32, device="cuda:0", generator=gen) for kk in (4096, 14336)}
        graphs = [capture([Gemv(QE.Q4_K, w, a8[kk], _lib.QMM_FLAG_ACT_Q8K) for w, (_, nn, kk) in zip(lw, PROJ)]) for lw in layers]
        dev_s, _ = time_graphs(graphs, 100, 10)
        sb = sum(alg_bytes(QE.Q4_K, mm, nn, kk) for _, nn, kk in PROJ)
        out[f"q4_k_act_q8k_m{mm}"] = {"us_per_step": round(dev_s * 1e6 / 100, 2), "GB/s": round(sb * 100 / dev_s / 1e9, 1)}
    # M = 4 with the shared-lhs projections grouped, as above
    a4g = {kk: torch.randn((4, kk), dtype=torch.float32, device="cuda:0", generator=gen) for kk in (4096, 14336)}
    graphs = [capture([GroupedGemv(QE.Q4_K, lw[0:3], a4g[4096]), Gemv(QE.Q4_K, lw[3], a4g[4096]),
                       GroupedGemv(QE.Q4_K, lw[4:6], a4g[4096]), Gemv(QE.Q4_K, lw[6], a4g[14336])]) for lw in layers]
    dev_s, _ = time_graphs(graphs, 100, 10)
    sb4 = sum(alg_bytes(QE.Q4_K, 4, nn, kk) for _, nn, kk in PROJ)
    out["q4_k_m4_grouped_4_launches"] = {"us_per_step": round(dev_s * 1e6 / 100, 2), "GB/s": round(sb4 * 100 / dev_s / 1e9, 1)}
    # M=4 over the same set
    if m == 1:
        acts4 = {k: torch.randn((4, k), dtype=torch.float32, device="cuda:0", generator=gen) for k in (4096, 14336)}
        graphs = [capture([Gemv(QE.Q4_K, w, acts4[k]) for w, (_, n, k) in zip(lw, PROJ)]) for lw in layers]
        dev_s, _ = time_graphs(graphs, 100, 10)
        b = sum(alg_bytes(QE.Q4_K, 4, n, k) for _, n, k in PROJ)
        out["q4_k_m4_GB/s"] = round(b * 100 / dev_s / 1e9, 1)
        # sixteen lhs rows, one step = the same seven projections (small-batch kernels)
        acts16 = {k: torch.randn((16, k), dtype=torch.float32, device="cuda:0", generator=gen) for k in (4096, 14336)}
        graphs = [capture([Gemv(QE.Q4_K, w, acts16[k]) for w, (_, n, k) in zip(lw, PROJ)]) for lw in layers]
        dev_s, _ = time_graphs(graphs, 100, 10)
        b = sum(alg_bytes(QE.Q4_K, 16, n, k) for _, n, k in PROJ)
        out["q4_k_m16"] = {"us_per_step": round(dev_s * 1e6 / 100, 2), "GB/s": round(b * 100 / dev_s / 1e9, 1)}
        del graphs
    # the decode kernel's asymptote: single Q4_K tensors of 196608 x 4096 (453 MB) and 393216 x 4096 (906 MB), beyond
    # every cache, M = 1; and the plain read of the same bytes
    if m == 1:
        for rows in (196608, 393216):
            wbig = make_weight(QE.Q4_K, rows, 4096, gen)
            mb = wbig.numel() // 1000000
            g = capture([Gemv(QE.Q4_K, wbig, acts[4096])])
            dev_s, _ = time_graphs([g], 10, 3)
            b = alg_bytes(QE.Q4_K, 1, rows, 4096)
            out[f"q4_k_m1_{rows}x4096_{mb}MB"] = {"us": round(dev_s * 1e6 / 10, 2), "GB/s": round(b * 10 / dev_s / 1e9, 1),
                                                  "frac_of_8000": round(b * 10 / dev_s / 1e9 / HBM_PEAK_GBS, 4)}
            g = capture([ReadProbe(wbig)])
            dev_s, _ = time_graphs([g], 10, 3)
            out[f"plain_read_{mb}MB"] = {"us": round(dev_s * 1e6 / 10, 2), "GB/s": round(wbig.numel() * 10 / dev_s / 1e9, 1)}
            del wbig, g
    # cfg4: Q6_K lm_head, M=1 (431 MB: larger than the cache by itself)
    w6 = make_weight(QE.Q6_K, 128256, 4096, gen)
    a1 = torch.randn((1, 4096), dtype=torch.float32, device="cuda:0", generator=gen)
    g = capture([Gemv(QE.Q6_K, w6, a1)])
    dev_s, _ = time_graphs([g], 20, 3)
    b = alg_bytes(QE.Q6_K, 1, 128256, 4096)
    out["q6_k_lm_head"] = {"us": round(dev_s * 1e6 / 20, 2), "GB/s": round(b * 20 / dev_s / 1e9, 1)}
    # ... and with 4 and 16 lhs rows (the small-batch matrix-core kernel: one pass over the weights for up to 16 rows)
    for mm in (4, 16):
        am = torch.randn((mm, 4096), dtype=torch.float32, device="cuda:0", generator=gen)
        g = capture([Gemv(QE.Q6_K, w6, am)])
        dev_s, _ = time_graphs([g], 10, 3)
        b = alg_bytes(QE.Q6_K, mm, 128256, 4096)
        out[f"q6_k_lm_head_m{mm}"] = {"us": round(dev_s * 1e6 / 10, 2), "GB/s": round(b * 10 / dev_s / 1e9, 1)}
    del w6
    # cfg5: Q4_K prefill, bf16 lhs [2048, 4096] x [14336, 4096]
    ab = torch.randn((2048, 4096), dtype=torch.float32, device="cuda:0", generator=gen).to(torch.bfloat16)
    wp = make_weight(QE.Q4_K, 14336, 4096, gen)
    g = capture([Gemv(QE.Q4_K, wp, ab)])
    dev_s, _ = time_graphs([g], 20, 3)
    us = dev_s * 1e6 / 20
    tf = 2 * 2048 * 14336 * 4096 / us / 1e6
    out["q4_k_prefill_m2048"] = {"us": round(us, 1), "TFLOP/s": round(tf, 1), "frac_of_2500": round(tf / BF16_PEAK_TFLOPS, 4)}
    del wp
    # the same shape with Q6_K and Q5_K weights (weights to fp16 integer planes, then a tile GEMM: the times include both)
    for enc, tag in ((QE.Q6_K, "q6_k_prefill_m2048"), (QE.Q5_K, "q5_k_prefill_m2048")):
        wk = make_weight(enc, 14336, 4096, gen)
        g = capture([Gemv(enc, wk, ab)])
        dev_s, _ = time_graphs([g], 10, 2)
        us = dev_s * 1e6 / 10
        tf = 2 * 2048 * 14336 * 4096 / us / 1e6
        out[tag] = {"us": round(us, 1), "TFLOP/s": round(tf, 1), "frac_of_2500": round(tf / BF16_PEAK_TFLOPS, 4)}
        del wk, g
    # cfg5, second weight set: GPTQ (group 128) prefill on the same shape
    wg = quantize_gptq(torch.randn((14336, 4096), dtype=torch.float32, device="cuda:0", generator=gen) * 0.02)
    g = capture([GptqMatmul(wg, ab)])
    dev_s, _ = time_graphs([g], 20, 3)
    us = dev_s * 1e6 / 20
    tf = 2 * 2048 * 14336 * 4096 / us / 1e6
    out["gptq_prefill_m2048"] = {"us": round(us, 1), "TFLOP/s": round(tf, 1), "frac_of_2500": round(tf / BF16_PEAK_TFLOPS, 4)}
    kept = RepackedGemv(QE.GPTQ, wg[:3], ab)
    dev_s, _ = time_graphs([capture([kept])], 20, 3)
    us = dev_s * 1e6 / 20
    tf = 2 * 2048 * 14336 * 4096 / us / 1e6
    out["gptq_prefill_m2048_repacked"] = {"us": round(us, 1), "TFLOP/s": round(tf, 1), "frac_of_2500": round(tf / BF16_PEAK_TFLOPS, 4)}
    del wg, kept
    # a prefill step of one layer: the seven Q4_K projections with 2048 / 512 lhs rows (bf16), as qmm_matmul calls and over
    # weight planes made once (qmm_repack; the planes of a layer take 0.5 GB)
    ws = [make_weight(QE.Q4_K, n, k, gen) for _, n, k in PROJ]
    for rows in (2048, 512):
        acts = {k: torch.randn((rows, k), dtype=torch.float32, device="cuda:0", generator=gen).to(torch.bfloat16) for k in (4096, 14336)}
        flops = sum(2.0 * rows * n * k for _, n, k in PROJ)
        res = {}
        qkv = torch.cat(ws[0:3])  # rows of packed blocks are independent: q | k | v as one matrix of 6144 rows
        for name, calls in (("qmm_matmul", [Gemv(QE.Q4_K, w, acts[k]) for w, (_, n, k) in zip(ws, PROJ)]),
                            ("qmm_matmul_repacked", [RepackedGemv(QE.Q4_K, (w,), acts[k]) for w, (_, n, k) in zip(ws, PROJ)]),
                            ("qmm_matmul_repacked_qkv_as_one_matrix", [RepackedGemv(QE.Q4_K, (qkv,), acts[4096])] +
                             [RepackedGemv(QE.Q4_K, (w,), acts[k]) for w, (_, n, k) in list(zip(ws, PROJ))[3:]])):
            dev_s, _ = time_graphs([capture(calls)], 10, 2)
            us = dev_s * 1e6 / 10
            res[name] = {"us_per_step": round(us, 1), "TFLOP/s": round(flops / us / 1e6, 1), "frac_of_2500": round(flops / us / 1e6 / BF16_PEAK_TFLOPS, 4)}
            del calls
        del qkv
        out[f"q4_k_prefill_layer_m{rows}"] = res
    del ws
    # cfg1 / cfg2: Q4_0 with Q8_0 activations
    for tag, mm, n, k, copies in (("q4_0_m1_4096x4096", 1, 4096, 4096, 32), ("q4_0_m16_14336x4096", 16, 14336, 4096, 10)):
        am = torch.randn((mm, k), dtype=torch.float32, device="cuda:0", generator=gen)
        cs = [Gemv(QE.Q4_0, make_weight(QE.Q4_0, n, k, gen), am) for _ in range(copies)]
        g = capture(cs)
        dev_s, _ = time_graphs([g], 20, 3)
        us = dev_s * 1e6 / (20 * copies)
        out[tag] = {"us": round(us, 3), "GB/s": round(alg_bytes(QE.Q4_0, mm, n, k) / us / 1e3, 1)}
        if mm == 1:  # the same launches with the RMS normalisation of the lhs as the kernel's prologue
            gamma = torch.ones((k,), dtype=torch.float32, device="cuda:0")
            g = capture([NormGemv(QE.Q4_0, c.w, am, gamma) for c in cs])
            dev_s, _ = time_graphs([g], 20, 3)
            out[tag + "_rmsnorm_prologue"] = {"us": round(dev_s * 1e6 / (20 * copies), 3)}
        del cs
    # GPTQ (group 128) decode on the gate shape
    am1 = torch.randn((1, 4096), dtype=torch.float32, device="cuda:0", generator=gen)
    cs = [GptqMatmul(quantize_gptq(torch.randn((14336, 4096), dtype=torch.float32, device="cuda:0", generator=gen) * 0.02),
                     am1) for _ in range(8)]
    g = capture(cs)
    dev_s, _ = time_graphs([g], 20, 3)
    us = dev_s * 1e6 / (20 * 8)
    out["gptq_g128_m1_14336x4096"] = {"us": round(us, 3), "GB/s": round((14336 * 4096 * 0.5176 + 4096 * 4 + 14336 * 4) / us / 1e3, 1)}
    # the same tensors read as an act-order checkpoint (desc_act=True): a random group for every k
    gi = torch.arange(4096, dtype=torch.int32, device="cuda:0")[torch.randperm(4096, device="cuda:0", generator=gen)] // 128
    g = capture([GptqMatmul(c.t, am1, g_idx=gi.to(torch.int32).contiguous()) for c in cs])
    dev_s, _ = time_graphs([g], 20, 3)
    us = dev_s * 1e6 / (20 * 8)
    out["gptq_g128_act_order_m1_14336x4096"] = {"us": round(us, 3), "GB/s": round((14336 * 4096 * 0.5176 + 4096 * 8 + 14336 * 4) / us / 1e3, 1)}
    # sixteen lhs rows: the small-batch matrix-core kernel
    am16 = torch.randn((16, 4096), dtype=torch.float32, device="cuda:0", generator=gen)
    g = capture([GptqMatmul(c.t, am16) for c in cs])
    dev_s, _ = time_graphs([g], 20, 3)
    us = dev_s * 1e6 / (20 * 8)
    out["gptq_g128_m16_14336x4096"] = {"us": round(us, 3), "GB/s": round((14336 * 4096 * 0.5176 + 16 * 4096 * 4 + 16 * 14336 * 4) / us / 1e3, 1)}
    del cs
    # Q5_K decode on the gate shape
    cs = [Gemv(QE.Q5_K, make_weight(QE.Q5_K, 14336, 4096, gen), am1) for _ in range(8)]
    g = capture(cs)
    dev_s, _ = time_graphs([g], 20, 3)
    us = dev_s * 1e6 / (20 * 8)
    out["q5_k_m1_14336x4096"] = {"us": round(us, 3), "GB/s": round(alg_bytes(QE.Q5_K, 1, 14336, 4096) / us / 1e3, 1)}
    # ... and with 8 fp32 / 16 bf16 lhs rows (one pass of the small-batch matrix-core kernel each)
    w5 = [c.w for c in cs]
    del cs
    for mm, dt, tag in ((8, torch.float32, "m8"), (16, torch.bfloat16, "m16_bf16")):
        am = torch.randn((mm, 4096), dtype=torch.float32, device="cuda:0", generator=gen).to(dt)
        g = capture([Gemv(QE.Q5_K, w_, am) for w_ in w5])
        dev_s, _ = time_graphs([g], 20, 3)
        us = dev_s * 1e6 / (20 * 8)
        out[f"q5_k_{tag}_14336x4096"] = {"us": round(us, 3)}
    del w5
    # Q4_0 prefill, same shape as cfg5: Q8_0 lhs codes and q - 8 as exact fp16 integers on the fp16 matrix cores (the time
    # includes the lhs quantisation and the weight plane conversion)
    ab32 = torch.randn((2048, 4096), dtype=torch.float32, device="cuda:0", generator=gen).to(torch.bfloat16)
    g = capture([Gemv(QE.Q4_0, make_weight(QE.Q4_0, 14336, 4096, gen), ab32)])
    dev_s, _ = time_graphs([g], 10, 2)
    us = dev_s * 1e6 / 10
    tf = 2 * 2048 * 14336 * 4096 / us / 1e6
    out["q4_0_prefill_m2048"] = {"us": round(us, 1), "TOP/s": round(tf, 1), "frac_of_2500": round(tf / BF16_PEAK_TFLOPS, 4)}
    del g, ab32
    # the headline's step in the other encodings (one fp32 row, seven qmm_matmul launches per layer, three layers rotated: more
    # than the last-level cache holds): what a model stored in that encoding pays per layer
    if m == 1:
        a1 = {kk: torch.randn((1, kk), dtype=torch.float32, device="cuda:0", generator=gen) for kk in (4096, 14336)}
        for enc, tag in ((QE.Q4_0, "q4_0"), (QE.Q6_K, "q6_k"), (QE.Q5_K, "q5_k"), (QE.GPTQ, "gptq_g128")):
            cs, sb = [], 0.0
            for _ in range(3):
                if enc == QE.GPTQ:
                    cs += [GptqMatmul(quantize_gptq(torch.randn((nn, kk), dtype=torch.float32, device="cuda:0", generator=gen) * 0.02), a1[kk])
                           for _, nn, kk in PROJ]
                else:
                    cs += [Gemv(enc, make_weight(enc, nn, kk, gen), a1[kk]) for _, nn, kk in PROJ]
            for _, nn, kk in PROJ:
                sb += (nn * kk * 0.5176 + 4 * kk + 4 * nn) if enc == QE.GPTQ else alg_bytes(enc, 1, nn, kk)
            # (one graph of two rotations, 42 kernel nodes: a host launch per step would be the limiter)
            dev_s, _ = time_graphs([capture(cs + cs)], 20, 3)
            out[f"{tag}_m1_seven_projections"] = {"us_per_step": round(dev_s * 1e6 / 120, 2), "GB/s": round(sb * 120 / dev_s / 1e9, 1)}
            del cs
    return out


if __name__ == "__main__":
    sys.exit(main())
