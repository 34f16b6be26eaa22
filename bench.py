"""Throughput of the packed batched-dots path on one MI355X, with its roofline and a CPU baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype i8] [--shape M N K] [--no-others] [--no-cpu]
                    [--no-vendor] [--no-ceiling]

One "step" is one packed product C = A * B^T over one synthetic batch (B is packed once, before the timed
region, as the reference's own benchmark does: bench/bench.hpp:238-255). The headline workload is the
i8 -> i32 product at M = N = K = 8192; bf16 and e4m3 at the same shape and the HBM-bound retrieval shape
(1024 queries x 1,048,576 vectors x 768) are measured the same way and reported under "others".
gso/s = 2*M*N*K / seconds / 1e9 (bench/bench.hpp:257). All operands are resident in HBM before timing.
Every step sits between two events of its own on the launch stream: `kernel_ms` is the mean over the timed region,
`kernel_ms_median` and `kernel_ms_min` come from the per-step pairs (include/numkong/dots/README.md:127-135 quotes
medians). `others` also holds, measured in the same process on the same box: the vendor library's GEMM on the same
operands (`vendor_*`: torch._int_mm / torch.matmul, which run hipBLASLt; timing only) and the rate an MFMA-only loop
sustains (`mfma_ceiling`, tests/probes/mfma_probes), so that a reader can tell the kernel from the part.

The symmetric kinds (`--metric symmetric`, `symmetric-angular`, `symmetric-euclidean`; N vectors of depth K, M is
ignored) time the whole call as the reference's benchmark does (bench/bench.hpp:397-438): packing the vectors,
building the tile list and the triangular product, into a workspace allocated once; they count N*(N+1)*K scalar
operations per call, the upper triangle only.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import queue
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published dense peaks, in T(FL)OP/s, for the MFMA the dtype runs on; HBM3E in GB/s.
MFMA_PEAK = {"i8": 5000.0, "u8": 5000.0, "bf16": 2500.0, "f16": 2500.0, "e4m3": 5000.0, "e5m2": 5000.0,
             "e2m3": 5000.0, "e3m2": 2500.0, "i4": 5000.0, "u4": 5000.0, "u1": 5000.0, "f32": 78.6, "f64": 78.6}
F16_ROUTE = ("e4m3", "e5m2")  # run widened to f16 on the f16 MFMA (2500): `frac` is against the fp8 peak, `frac_f16` against the instruction's
MFMA_NOTE = {"e4m3": "widened to f16 (the fp8 MFMA keeps 14 bits of a lane's sums): frac is against the fp8 peak of 5000, frac_f16 against the f16 MFMA it runs on",
             "e5m2": "widened to f16 (the fp8 MFMA keeps 14 bits of a lane's sums): frac is against the fp8 peak of 5000, frac_f16 against the f16 MFMA it runs on",
             "e2m3": "as i8 values eight times as large (exact), priced against the i8 MFMA peak", "e3m2": "widened to f16, priced against the f16 MFMA peak",
             "i4": "widened to i8, priced against the i8 MFMA peak", "u4": "widened to i8, priced against the i8 MFMA peak",
             "u1": "bits widened to i8 zeros and ones, priced against the i8 MFMA peak",
             "f32": "exact f32 products summed in f64 on the f64 MFMA (78.6 TFLOP/s), four sums per output as in the reference",
             "f64": "compensated f64 sums on the vector units: 10 f64 instructions per multiply-add, priced as the 2 flops of one"}
HBM_PEAK = 8000.0
# HBM-side bytes per launch (L2 <-> fabric) from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of `bench.py --probe`,
# each scaled by what the same counter reads for a 1 GiB elementwise kernel (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000);
# kept, with the commands, in profiles/traffic.json. Not re-measured by a plain run: counters need the profiler.
def measured_traffic(*key):
    global _TRAFFIC
    if _TRAFFIC is None:
        try:
            with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
                _TRAFFIC = json.load(f)["bytes_per_launch"]
        except (OSError, ValueError, KeyError):
            _TRAFFIC = {}
    return _TRAFFIC.get("_".join(str(part) for part in key))


_TRAFFIC = None
HEADLINE = ("i8", 8192, 8192, 8192)
METRIC_DTYPES = ("i8", "bf16", "e4m3")  # the three types BASELINE's metric names, all at the headline shape
OTHERS = [("bf16", 8192, 8192, 8192, "dots"), ("e4m3", 8192, 8192, 8192, "dots"), ("e5m2", 8192, 8192, 8192, "dots"),
          ("f16", 8192, 8192, 8192, "dots"), ("i8", 8192, 8191, 1000, "dots"), ("f16", 8192, 8191, 1000, "dots"),
          ("bf16", 4096, 4096, 4096, "dots"), ("i8", 2048, 2048, 2048, "dots"),
          ("i8", 1024, 1 << 20, 768, "dots"), ("u8", 1024, 1 << 20, 768, "dots"),
          ("i8", 1024, 1 << 20, 768, "angular"), ("i8", 8192, 8192, 8192, "symmetric"), ("bf16", 8192, 8192, 8192, "symmetric"),
          ("i4", 8192, 8192, 8192, "dots"), ("e2m3", 8192, 8192, 8192, "dots"), ("u1", 8192, 8192, 8192, "dots"),
          ("f32", 4096, 4096, 4096, "dots"), ("f64", 4096, 4096, 4096, "dots")]
VENDOR = [("i8", 8192, 8192, 8192), ("bf16", 8192, 8192, 8192), ("f16", 8192, 8192, 8192)]
KINDS = {"angular": ord("N"), "euclidean": ord("E")}  # nk_kernel_angulars_packed_k, nk_kernel_euclideans_packed_k
# nk_kernel_dots_symmetric_k, nk_kernel_angulars_symmetric_k, nk_kernel_euclideans_symmetric_k
SYMMETRIC_KINDS = {"symmetric": ord("y"), "symmetric-angular": ord("n"), "symmetric-euclidean": ord("D")}


def make_operands(dtype, m, n, k, seed=42):
    """Synthetic inputs of BASELINE's families, generated on the GPU: ints uniform over the full range, bf16 N(0,1),
    f16 log-normal(0,1) magnitudes with random signs, fp8 N(0,1) scaled to half the largest finite value with 1 %
    zeros (clamped to the finite range before the cast: e5m2's literal configuration overflows to Inf and is almost
    all NaN, which the parity tests cover)."""
    import torch

    g = torch.Generator(device="cuda:0").manual_seed(seed)
    def one(rows):
        if dtype in ("i4", "u4"):  # two 4-bit values per byte, every byte value
            return torch.randint(0, 256, (rows, (k + 1) // 2), dtype=torch.uint8, device="cuda:0", generator=g)
        if dtype in ("f32", "f64"):
            return torch.randn((rows, k), device="cuda:0", generator=g, dtype=torch.float32 if dtype == "f32" else torch.float64)
        if dtype == "u1":  # eight bits per byte
            return torch.randint(0, 256, (rows, (k + 7) // 8), dtype=torch.uint8, device="cuda:0", generator=g)
        if dtype in ("e2m3", "e3m2"):  # every 6-bit code is a finite number
            return torch.randint(0, 64, (rows, k), dtype=torch.uint8, device="cuda:0", generator=g)
        if dtype == "i8":
            return torch.randint(-128, 128, (rows, k), dtype=torch.int8, device="cuda:0", generator=g)
        if dtype == "u8":
            return torch.randint(0, 256, (rows, k), dtype=torch.uint8, device="cuda:0", generator=g)
        z = torch.randn((rows, k), device="cuda:0", generator=g)
        if dtype == "bf16":
            return z.to(torch.bfloat16).view(torch.int16)
        if dtype == "f16":
            sign = torch.randint(0, 2, (rows, k), device="cuda:0", generator=g).float() * 2 - 1
            return (torch.exp(z) * sign).to(torch.float16).view(torch.int16)
        top = 448.0 if dtype == "e4m3" else 57344.0
        z = (z * (0.5 * top)).clamp(-top, top)  # torch's cast has no saturation: clamp first
        z = z * (torch.rand((rows, k), device="cuda:0", generator=g) >= 0.01)
        return z.to(torch.float8_e4m3fn if dtype == "e4m3" else torch.float8_e5m2).view(torch.uint8)
    return one(m), one(n)


# From idle the part takes some tens of milliseconds of load to reach the clocks it then holds (measured, first series of
# a process against the same series later in it: bf16 4096^3 144 against 120 us per launch, i8 8192^3 455 against 417),
# and a short series timed from idle reads that ramp instead of the kernel. Every timing here, this library's kernels
# and the vendor library's alike, is therefore preceded by this much untimed running of the same step (--spin-up-ms;
# 0 turns it off); the warm-up steps and the timed steps follow as asked for.
SPIN_UP_MS = 100.0


def timed_steps(step, steps, warmup):
    """Untimed running of `step` until the clocks have settled (SPIN_UP_MS), `warmup` untimed calls, then `steps` timed
    ones, each between two events of its own on torch's current stream (the stream the kernels are launched on). Returns
    wall ms per step and the device times in ms: mean over the whole region, median and minimum of the per-step pairs."""
    import torch

    if SPIN_UP_MS > 0:
        until = time.perf_counter() + SPIN_UP_MS * 1e-3
        while time.perf_counter() < until:
            for _ in range(4):
                step()
            torch.cuda.synchronize()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    wall = time.perf_counter()
    marks[0].record()
    for at in range(steps):
        step()
        marks[at + 1].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - wall) * 1e3 / steps
    each = sorted(marks[at].elapsed_time(marks[at + 1]) for at in range(steps))
    median = each[steps // 2] if steps % 2 else 0.5 * (each[steps // 2 - 1] + each[steps // 2])
    return wall, {"kernel_ms": marks[0].elapsed_time(marks[steps]) / steps, "kernel_ms_median": median, "kernel_ms_min": each[0]}


def timed_graph(step, steps):
    """Device time per launch of a short kernel: `steps` launches recorded into one HIP graph and replayed, so that the
    host's launch rate (a Python call and a launch take about as long as a 10 us kernel runs) is not what is read.
    Replayed untimed until the clocks have settled, then timed over 5 replays: mean, median and minimum per launch."""
    import torch

    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        for _ in range(steps):
            step()
    until = time.perf_counter() + max(SPIN_UP_MS, 20.0) * 1e-3
    while time.perf_counter() < until:
        graph.replay()
        torch.cuda.synchronize()
    each = []
    for _ in range(5):
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        graph.replay()
        end.record()
        torch.cuda.synchronize()
        each.append(begin.elapsed_time(end) / steps)
    each.sort()
    return {"kernel_ms": sum(each) / len(each), "kernel_ms_median": each[len(each) // 2], "kernel_ms_min": each[0]}


def time_symmetric(dtype, n, k, steps, warmup, metric):
    """All pairs of n vectors of depth k, upper triangle: one call packs, lists its tiles and multiplies."""
    import torch

    import numkong_amd as nk
    from numkong_amd import api

    lib = nk.library()
    vectors, _ = make_operands(dtype, n, 1, k)
    code, row_bytes = api.DTYPES[dtype][0], vectors.shape[1] * vectors.element_size()
    result = torch.zeros((n, n), dtype=torch.int32 if dtype in ("i8", "u8") and metric == "symmetric" else torch.float32,
                         device="cuda:0")
    workspace_bytes = lib.nk_amd_symmetric_workspace_size(code, n, k, 0, n)
    workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        status = lib.nk_amd_symmetric_async(SYMMETRIC_KINDS[metric], code, vectors.data_ptr(), n, k, row_bytes,
                                            result.data_ptr(), n * 4, 0, n, workspace.data_ptr(), workspace_bytes, stream)
        if status:
            raise RuntimeError(lib.nk_hip_last_error().decode())

    wall, times = timed_steps(step, steps, warmup)
    device_ms = times["kernel_ms"]
    ops = 1.0 * n * (n + 1) * k
    achieved = ops / (device_ms * 1e-3) / 1e12
    out = {"ms_per_step": wall, **times, "gso_per_s": ops / (wall * 1e-3) / 1e9,
           "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_PEAK[dtype], "unit": "TFLOP/s",
                        "frac": achieved / MFMA_PEAK[dtype], "traffic": measured_traffic(dtype, n, n, k, metric),
                        "note": "whole call (pack + tile list + product) over the operations of the upper triangle"}}
    del vectors, result, workspace
    torch.cuda.empty_cache()
    return out


PACKS = [("i8", 8192, 8192), ("bf16", 8192, 8192), ("i8", 1 << 20, 768), ("f32", 4096, 4096)]


def time_pack(dtype, n, k, steps, warmup):
    """nk_dots_pack alone (every kernel it launches): B read once, its image written once, so HBM bounds it."""
    import torch

    import numkong_amd as nk
    from numkong_amd import api

    lib = nk.library()
    b = make_operands(dtype, 1, n, k)[1]
    size = api.dots_packed_size(dtype, n, k)
    image = torch.empty(size, dtype=torch.uint8, device="cuda:0")
    code, row_bytes = api.DTYPES[dtype][0], b.shape[1] * b.element_size()
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        if lib.nk_amd_dots_pack_async(code, b.data_ptr(), n, k, row_bytes, image.data_ptr(), stream):
            raise RuntimeError(lib.nk_hip_last_error().decode())

    _, times = timed_steps(step, steps, warmup)
    device_ms = times["kernel_ms"]
    algorithmic = n * row_bytes + size
    del b, image
    torch.cuda.empty_cache()
    return {**times, "roofline": {"bound": "hbm", "achieved": algorithmic / (device_ms * 1e-3) / 1e9, "peak": HBM_PEAK,
                                                 "unit": "GB/s", "frac": algorithmic / (device_ms * 1e-3) / 1e9 / HBM_PEAK, "traffic": None,
                                                 "note": f"{n * row_bytes} bytes of B read + {size} bytes of image written"}}


def time_gpu(dtype, m, n, k, steps, warmup, metric="dots"):
    import torch

    import numkong_amd as nk
    from numkong_amd import api

    if metric in SYMMETRIC_KINDS:
        return time_symmetric(dtype, n, k, steps, warmup, metric)
    lib = nk.library()
    a, b = make_operands(dtype, m, n, k)
    packed = nk.dots_pack(b, dtype)
    del b
    wide = dtype in ("f32", "f64")  # f64 results
    c = torch.empty((m, n), dtype=torch.float64 if wide else (torch.int32 if dtype in ("i8", "u8") and metric == "dots" else torch.float32),
                    device="cuda:0")
    code, row_bytes = api.DTYPES[dtype][0], a.shape[1] * a.element_size()

    def step():
        stream = torch.cuda.current_stream().cuda_stream  # the kernel is launched on this stream, so torch events see it
        if metric == "dots":
            status = lib.nk_amd_dots_packed_async(code, a.data_ptr(), packed.buffer.data_ptr(), c.data_ptr(), m, n, k,
                                                  row_bytes, n * c.element_size(), stream)
        else:  # the same product with the distance finaliser fused into its epilogue
            status = lib.nk_amd_spatials_packed_async(KINDS[metric], code, a.data_ptr(), packed.buffer.data_ptr(), c.data_ptr(),
                                                      m, n, k, row_bytes, n * 4, stream)
        if status:
            raise RuntimeError(lib.nk_hip_last_error().decode())

    wall, times = timed_steps(step, steps, warmup)
    timed_as = None
    if times["kernel_ms"] < 0.06:  # shorter than a few launches' worth of host time: the events read the host's pace
        times, timed_as = timed_graph(step, steps), f"{steps} launches recorded into one HIP graph, 5 replays (the events around single launches read the host's launch rate: {times['kernel_ms'] * 1e3:.1f} us per launch)"
    device_ms = times["kernel_ms"]
    ops = 2.0 * m * n * k
    result = {"ms_per_step": wall, **times, "gso_per_s": ops / (wall * 1e-3) / 1e9}
    if timed_as:
        result["timed_as"] = timed_as
    if m * n >= 64 * k * 8 and dtype in ("i8", "u8") and n >= 1 << 18:  # retrieval shape: HBM-bound on C and the packed stream
        algorithmic = (m + n) * row_bytes + m * n * 4
        result["roofline"] = {"bound": "hbm", "achieved": algorithmic / (device_ms * 1e-3) / 1e9, "peak": HBM_PEAK,
                              "unit": "GB/s", "frac": algorithmic / (device_ms * 1e-3) / 1e9 / HBM_PEAK,
                              "traffic": measured_traffic(*((dtype, m, n, k) if metric == "dots" else (dtype, m, n, k, metric)))}
    else:
        achieved = ops / (device_ms * 1e-3) / 1e12
        result["roofline"] = {"bound": "mfma", "achieved": achieved, "peak": MFMA_PEAK[dtype], "unit": "TFLOP/s",
                              "frac": achieved / MFMA_PEAK[dtype],
                              "traffic": measured_traffic(*((dtype, m, n, k) if metric == "dots" else (dtype, m, n, k, metric)))}
        if dtype in F16_ROUTE:
            result["roofline"]["frac_f16"] = achieved / MFMA_PEAK["f16"]
        if dtype in MFMA_NOTE:
            result["roofline"]["note"] = MFMA_NOTE[dtype]
    del a, packed, c
    torch.cuda.empty_cache()
    return result


def time_sync_abi(dtype, m, n, k, calls=200):
    """The reference-ABI symbol itself (`nk_dots_packed_<T>`: synchronous, pointers classified per call) on operands in
    device memory: wall-clock per call, next to the device time of the same product through the asynchronous entry
    point, so that what the drop-in symbol adds to a launch is a number."""
    import torch

    import numkong_amd as nk
    from numkong_amd import api

    lib = nk.library()
    a, b = make_operands(dtype, m, n, k)
    packed = nk.dots_pack(b, dtype)
    c = torch.empty((m, n), dtype=torch.int32 if dtype in ("i8", "u8") else torch.float32, device="cuda:0")
    code, row_bytes = api.DTYPES[dtype][0], a.shape[1] * a.element_size()
    stream = torch.cuda.current_stream().cuda_stream
    entry = getattr(lib, f"nk_dots_packed_{dtype}")
    arguments = (a.data_ptr(), packed.buffer.data_ptr(), c.data_ptr(), m, n, k, row_bytes, n * 4)
    for _ in range(20):
        entry(*arguments)
    torch.cuda.synchronize()
    begin = time.perf_counter()
    for _ in range(calls):
        entry(*arguments)
    sync_us = (time.perf_counter() - begin) * 1e6 / calls
    if lib.nk_amd_last_error():
        raise RuntimeError(lib.nk_amd_last_error().decode())

    def step():
        if lib.nk_amd_dots_packed_async(code, *arguments, stream):
            raise RuntimeError(lib.nk_hip_last_error().decode())

    _, times = timed_steps(step, calls, 20)
    # the same asynchronous launch followed by a wait for it, as a caller of the synchronous symbol would otherwise write
    begin = time.perf_counter()
    for _ in range(calls):
        step()
        torch.cuda.current_stream().synchronize()
    launch_and_wait_us = (time.perf_counter() - begin) * 1e6 / calls
    del a, packed, c
    torch.cuda.empty_cache()
    return {"sync_wall_us_per_call": sync_us, "async_kernel_us": times["kernel_ms"] * 1e3,
            "async_launch_and_wait_us": launch_and_wait_us, "sync_minus_kernel_us": sync_us - times["kernel_ms"] * 1e3,
            "what": f"nk_dots_packed_{dtype} on device pointers, {calls} calls back to back, wall-clock per call; "
                    "nk_amd_dots_packed_async's device time per launch; the asynchronous launch plus a stream wait, wall-clock"}


def time_vendor(dtype, m, n, k, steps, warmup):
    """The vendor library's GEMM (hipBLASLt through torch) on operands of the same family in the same process: what
    this part gives a tuned kernel of the same shape. Timing only; nothing of it is used by the product."""
    import torch

    a, b = make_operands(dtype, m, n, k)
    if dtype == "i8":
        bt = b.t()  # (k x n) view of the row-major B: the library picks its own transposed kernel
        step = lambda: torch._int_mm(a, bt)
    else:
        view = torch.bfloat16 if dtype == "bf16" else torch.float16
        av, bt = a.view(view), b.view(view).t()
        step = lambda: torch.matmul(av, bt)
    _, times = timed_steps(step, steps, warmup)
    achieved = 2.0 * m * n * k / (times["kernel_ms"] * 1e-3) / 1e12
    del a, b
    torch.cuda.empty_cache()
    return {**times, "tops": achieved, "frac": achieved / MFMA_PEAK[dtype],
            "what": "torch._int_mm (i8 -> i32)" if dtype == "i8" else f"torch.matmul ({dtype} -> {dtype}, f32 accumulation)"}


def mfma_ceiling():
    """The rate an MFMA-only loop sustains on this box (tests/probes/mfma_probes ceiling), as a child process."""
    import subprocess

    probe = os.path.join(ROOT, "tests", "probes", "mfma_probes")
    if not os.path.exists(probe):
        return {"error": "tests/probes/mfma_probes is not built"}
    try:
        done = subprocess.run([probe, "ceiling", "--json"], capture_output=True, text=True, timeout=120)
        return json.loads(done.stdout) if done.returncode == 0 else {"error": done.stderr[-300:]}
    except (OSError, ValueError, subprocess.TimeoutExpired) as failure:
        return {"error": str(failure)}


def cpu_baseline(dtype, m, n, k, budget_rows=8192):
    """The reference's own dots path on the host cores: B packed once, A split into 64-row tiles handed out
    dynamically to one thread per core (python/matrix.c:466-483, python/matrix.h:18), best-dispatch kernel.
    Falls back to this repository's scalar oracle on a smaller sample if the reference build is absent."""
    import numpy as np

    from tests import support

    oracle = support.load_oracle()
    reference = support.load_reference()
    rng = np.random.default_rng(42)
    allowed = sorted(os.sched_getaffinity(0))  # every core this process may run on, one pinned thread each
    cores = max(1, len(allowed))
    if reference is None:
        rows, cols = 16, min(n, 256)
        a = support.random_matrix(oracle, dtype, rows, k, rng)
        b = support.random_matrix(oracle, dtype, cols, k, rng)
        start = time.perf_counter()
        oracle.dots_packed(dtype, a, b)
        seconds = time.perf_counter() - start
        return {"value": 2.0 * rows * cols * k / seconds / 1e9, "unit": "gso/s", "cores": 1, "kind": "port",
                "sample": f"{rows} x {cols} x {k} of the workload, scalar restatement (reference build not present)"}
    rows = min(m, budget_rows)
    a = support.random_matrix(oracle, dtype, rows, k, rng)
    b = support.random_matrix(oracle, dtype, min(n, 8192), k, rng)
    cols = b.shape[0]
    viable = reference.capabilities
    size_fn, _ = reference.kernel(support.KIND_SIZE, dtype, viable)
    pack_fn, _ = reference.kernel(support.KIND_PACK, dtype, viable)
    dots_fn, used = reference.kernel(support.KIND_PACKED, dtype, viable)
    packed = np.zeros(int(size_fn(cols, k)) + 64, np.uint8)
    pack_fn(b.ctypes.data, cols, k, b.strides[0], packed.ctypes.data)
    c = np.empty((rows, cols), support.OUTPUT[dtype])
    tile = 64

    def run_once():
        tiles: "queue.SimpleQueue[int]" = queue.SimpleQueue()
        for start in range(0, rows, tile):
            tiles.put(start)

        def worker(cpu):
            try:
                os.sched_setaffinity(0, {cpu})  # (0 = the calling thread)
            except OSError:
                pass
            reference.lib.nk_configure_thread(ctypes.c_uint64(viable))
            while True:
                try:
                    start = tiles.get_nowait()
                except queue.Empty:
                    return
                count = min(tile, rows - start)
                dots_fn(a.ctypes.data + start * a.strides[0], packed.ctypes.data, c.ctypes.data + start * c.strides[0],
                        count, cols, k, a.strides[0], c.strides[0])

        threads = [threading.Thread(target=worker, args=(cpu,)) for cpu in allowed]
        begin = time.perf_counter()
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        return time.perf_counter() - begin

    run_once()
    runs = sorted(run_once() for _ in range(3))
    best, median = runs[0], runs[1]
    return {"value": 2.0 * rows * cols * k / best / 1e9, "median": 2.0 * rows * cols * k / median / 1e9, "unit": "gso/s",
            "cores": cores, "online_cores": os.cpu_count(), "kind": "reference", "kernel_capability": hex(used),
            "sample": (f"{rows} rows of A x {cols} packed rows of B x depth {k}, 64-row tiles handed to {cores} pinned threads "
                       "(every core the process may use), best and median of 3 after a warm-up run")}


def main():
    global SPIN_UP_MS
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--dtype", default=HEADLINE[0])
    parser.add_argument("--shape", type=int, nargs=3, default=list(HEADLINE[1:]))
    parser.add_argument("--metric", default="dots", choices=["dots", "angular", "euclidean"] + sorted(SYMMETRIC_KINDS),
                        help="what the timed call computes: the packed product, one of the packed distances on top of it, or "
                             "one of the symmetric kinds over N vectors of depth K")
    parser.add_argument("--spin-up-ms", type=float, default=SPIN_UP_MS,
                        help="untimed running of each timed step before its warm-up steps, until the clocks have settled (0: none)")
    parser.add_argument("--no-others", action="store_true")
    parser.add_argument("--no-cpu", action="store_true")
    parser.add_argument("--no-vendor", action="store_true", help="skip the vendor GEMM timings (others.vendor_*)")
    parser.add_argument("--no-ceiling", action="store_true", help="skip the MFMA-only loop (others.mfma_ceiling)")
    parser.add_argument("--vendor-probe", action="store_true",
                        help="for rocprofv3 runs: the vendor library's GEMM for --dtype (i8, bf16, f16) and --shape, 10 launches after 5, nothing else")
    parser.add_argument("--probe", action="store_true",
                        help="for rocprofv3 --pmc runs: launch a plain 1 GiB elementwise copy kernel 3 times, then the selected product 3 times, nothing else")
    args = parser.parse_args()
    SPIN_UP_MS = 0.0 if args.probe or args.vendor_probe else max(0.0, args.spin_up_ms)
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU leg (rows of A or of B shard without "
                 "communication); run with --gpus 1")
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    m, n, k = args.shape
    if args.vendor_probe:
        print(json.dumps({f"vendor_{args.dtype}_{m}x{n}x{k}": time_vendor(args.dtype, m, n, k, 10, 5)}))
        return
    if args.probe:
        source = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").fill_(1)
        target = torch.empty_like(source)
        for _ in range(3):
            torch.add(source, 1, out=target)  # an elementwise kernel of known traffic: 1 GiB read + 1 GiB written
        torch.cuda.synchronize()
        del source, target
        time_gpu(args.dtype, m, n, k, 3, 0, args.metric)
        return
    head = time_gpu(args.dtype, m, n, k, args.steps, args.warmup, args.metric)
    headline = (args.dtype, m, n, k, args.metric) == (*HEADLINE, "dots")
    # The metric names three types at 8192^3: all three are timed with the full step count, and their figures ride
    # inside `roofline` and `cpu_baseline` (`by_dtype`), next to the headline's.
    def brief(r):
        keep = {"kernel_ms": r["kernel_ms"], "kernel_ms_median": r["kernel_ms_median"], "kernel_ms_min": r["kernel_ms_min"],
                "achieved": r["roofline"]["achieved"], "peak": r["roofline"]["peak"], "frac": r["roofline"]["frac"],
                "traffic": r["roofline"]["traffic"]}
        if "frac_f16" in r["roofline"]:
            keep["frac_f16"] = r["roofline"]["frac_f16"]
        return keep

    metric_types = {}
    if headline:
        metric_types["i8"] = head
        for dtype in METRIC_DTYPES[1:]:
            metric_types[dtype] = time_gpu(dtype, m, n, k, args.steps, args.warmup, "dots")
        head["roofline"]["by_dtype"] = {dtype: brief(r) for dtype, r in metric_types.items()}
    line = {}
    # (`others` goes first: it is long, and what a reader of the end of the line looks for comes after it)
    if not args.no_others:
        line["others"] = {}
        for dtype, om, on, ok, metric in OTHERS:
            if (dtype, om, on, ok, metric) in [(t, m, n, k, "dots") for t in metric_types]:
                r = metric_types[dtype]
            else:
                r = time_gpu(dtype, om, on, ok, max(3, args.steps // 2), max(2, args.warmup // 2), metric)
            name = f"{dtype}_{on}x{ok}_{metric}" if metric in SYMMETRIC_KINDS else f"{dtype}_{om}x{on}x{ok}" + ("" if metric == "dots" else "_" + metric)
            line["others"][name] = {"gso_per_s": r["gso_per_s"], "kernel_ms": r["kernel_ms"], "kernel_ms_median": r["kernel_ms_median"],
                                    "kernel_ms_min": r["kernel_ms_min"], "roofline": {key: value for key, value in r["roofline"].items() if key != "by_dtype"}}
            if "timed_as" in r:
                line["others"][name]["timed_as"] = r["timed_as"]
        for dtype, on, ok in PACKS:
            line["others"][f"pack_{dtype}_{on}x{ok}"] = time_pack(dtype, on, ok, max(3, args.steps // 2), max(2, args.warmup // 2))
        line["others"]["sync_abi_i8_2048"] = time_sync_abi("i8", 2048, 2048, 2048)
    if not args.no_vendor:
        line.setdefault("others", {})
        for dtype, om, on, ok in VENDOR:
            line["others"][f"vendor_{dtype}_{om}x{on}x{ok}"] = time_vendor(dtype, om, on, ok, max(3, args.steps // 2), max(2, args.warmup // 2))
    if not args.no_ceiling:
        line.setdefault("others", {})["mfma_ceiling"] = mfma_ceiling()
    if headline and "others" in line:
        # Boxes of one pool differ by 15 % on power-bound kernels: the same run's MFMA-only loop and the vendor library's
        # GEMM are the yardsticks that move with the box.
        forms = line["others"].get("mfma_ceiling", {}).get("forms", {})
        probe_form = {"i8": "i8 32x32x32, random", "bf16": "bf16 32x32x16, random", "e4m3": "f16 32x32x16 on e4m3 values, random"}
        same_run = {}
        for dtype, r in metric_types.items():
            entry = {}
            if probe_form[dtype] in forms:
                entry["over_mfma_only_loop"] = r["roofline"]["achieved"] / forms[probe_form[dtype]]["tops"]
            vendor = line["others"].get(f"vendor_{dtype}_{m}x{n}x{k}")
            if vendor:
                entry["over_vendor_gemm"] = r["roofline"]["achieved"] / vendor["tops"]
            if entry:
                same_run[dtype] = entry
        if same_run:
            head["roofline"]["same_run"] = same_run
    line.update({
        "metric": "gso/s and % MFMA peak: i8->i32, bf16->f32, e4m3->f32 packed dots at 8192^3",
        "value": head["gso_per_s"], "unit": "gso/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": (f"{args.dtype} {args.metric} all pairs of N={n} vectors of depth K={k}, upper triangle, vectors "
                                "row-major in HBM, packed inside the timed call") if args.metric in SYMMETRIC_KINDS else
                               (f"{args.dtype} packed {args.metric} C = A * B^T, M={m} N={n} K={k}, A row-major in HBM, "
                                "B packed once outside the timed region, C overwritten")},
        "kernel_ms": head["kernel_ms"], "kernel_ms_median": head["kernel_ms_median"], "kernel_ms_min": head["kernel_ms_min"],
        "spin_up_ms": SPIN_UP_MS,  # untimed running before the warm-up steps of every timing (clock ramp from idle)
        "roofline": head["roofline"],
    })
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args.dtype, m, n, k)
        if headline:  # the metric's other two types, on a stated share of the rows of A (the kernels are 5-10 times slower)
            line["cpu_baseline"]["by_dtype"] = {"i8": {key: line["cpu_baseline"][key] for key in ("value", "median", "cores", "kernel_capability", "sample")}}
            for dtype in METRIC_DTYPES[1:]:
                other = cpu_baseline(dtype, m, n, k, budget_rows=2048)
                line["cpu_baseline"]["by_dtype"][dtype] = {key: other[key] for key in ("value", "median", "cores", "kernel_capability", "sample") if key in other}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
