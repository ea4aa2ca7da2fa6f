#!/usr/bin/env python3
"""Throughput of the quantize/dequantize path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg5] [--no-sweep] [--no-cpu]

A step = one pass of the hot path over one synthetic tensor that is already
resident in HBM: fused dynamic quantize (abs-max, scale, round, clamp, pack)
followed by dequantize of the result.  Launches rotate through independent buffer
sets (>= 1 GiB in total) so that no launch finds its operands in the 256 MB
Infinity Cache from an earlier launch.  The headline workload is the largest
configuration (cfg5: e2m1 block 32, bf16 [28672, 8192]); the other four
configurations are measured in short loops and reported under "per_config"
(launches shorter than 16 us also as a replayed HIP graph, "graph_replay_ms":
the host's share of an eager call bounds them).

value      = algorithmic bytes of one step / wall time per step  (GB/s, 1e9)
             algorithmic bytes = input once + codes once + scales once, per direction
roofline   = the quantize kernel alone: algorithmic bytes / its launch duration, against the 8 TB/s HBM peak.
             Duration = the median over 50 regions of back-to-back launches, each between two HIP events on
             the launch stream (timed_median); the average over one region of K launches stands beside it.
             roofline.per_config holds the same fraction for the three launches of every configuration
cpu_baseline = the CPU oracle (oracle/cq_oracle.c, the scalar restatement of the
             reference algorithm) on a bounded row sample of the same tensor, best of three
             runs on every hardware thread the job may use
inputs     = generated on the host with numpy's PCG64 (make_input), uploaded, rounded to the tensor's type
memory     = buffers are dropped between the cases but never handed back to the driver (no empty_cache):
             tensors allocated out of memory that the process had released and mapped again made the larger
             matrix-vector launches 10 % slower (37.1 against 33.5 us) and the other kernels 0-3 %

Prints ONE JSON line on stdout.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# name -> (rows, cols, elem, value, block, generator)
WORKLOADS = {
    "cfg1": dict(shape=(1024, 1024), elem="F32", value="Q8S", block=None, dist="normal1", seed=1,
                 desc="per-tensor symmetric q8, f32 [1024,1024] ~N(0,1)"),
    "cfg2": dict(shape=(4096, 4096), elem="BF16", value="Q8S", block=32, dist="normal_outliers", seed=2,
                 desc="per-block(32) symmetric q8, bf16 [4096,4096] ~N(0,0.02) + 0.1% x50 outliers"),
    "cfg3": dict(shape=(14336, 4096), elem="BF16", value="Q4S", block=32, dist="normal", seed=3,
                 desc="per-block(32) symmetric q4, bf16 [14336,4096] ~N(0,0.02)"),
    "cfg4": dict(shape=(8192, 8192), elem="F32", value="Q2S", block=64, dist="laplace", seed=4,
                 desc="per-block(64) symmetric q2, f32 [8192,8192] ~Laplace(0,0.01)"),
    "cfg5": dict(shape=(28672, 8192), elem="BF16", value="E2M1", block=32, dist="normal_t3", seed=5,
                 desc="per-block(32) e2m1 (4-bit fields), bf16 [28672,8192] ~N(0,0.02) + 1% Student-t(3)"),
}

def measured_traffic():
    """HBM bytes per launch (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, calibrated on a copy of known size) of the
    three kernels of every configuration, as recorded in profiles/traffic.json; {} when the file is absent."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return {}
    with open(path) as f:
        return json.load(f).get("hbm_bytes_per_launch", {})


def algorithmic_bytes(w) -> int:
    rows, cols = w["shape"]
    n = rows * cols
    elem_bytes = 4 if w["elem"] == "F32" else 2
    bits = {"Q8S": 8, "Q4S": 4, "Q2S": 2, "E2M1": 4}[w["value"]]
    scales = 1 if w["block"] is None else n // w["block"]
    return n * elem_bytes + n * bits // 8 + scales * 4


GEN_CHUNK_ELEMS = 1 << 24  # the host generator draws whole rows, this many elements at a time


def make_input(torch, w):
    """The seeded synthetic tensor of a configuration, generated on the HOST and uploaded, so that the bytes do
    not depend on the GPU or on the torch version.

    Generator: numpy.random.Generator(numpy.random.PCG64(seed)), seed = the configuration's number.  The
    tensor is produced in chunks of max(1, 2^24 // cols) whole rows, first row first; per chunk, in this
    order of draws (n = elements of the chunk, all float32):
      normal1          z = standard_normal(n)                                   x = z
      normal           z = standard_normal(n)                                   x = 0.02 z
      normal_outliers  z = standard_normal(n); u = random(n)                    x = 0.02 z * (50 if u < 0.001 else 1)
      laplace          u = random(n) - 0.5                                      x = -0.01 sign(u) log1p(-2 min(|u|, 0.4999999))
      normal_t3        z = standard_normal(n); u = random(n);
                       t = standard_t(3, size = number of u < 0.01)             x = 0.02 t where u < 0.01, else 0.02 z
    The float32 chunk is copied to the device and rounded there to the tensor's type (round to nearest even)."""
    import numpy as np

    rows, cols = w["shape"]
    rng = np.random.Generator(np.random.PCG64(w["seed"]))
    dt = torch.float32 if w["elem"] == "F32" else torch.bfloat16
    out = torch.empty((rows, cols), dtype=dt, device="cuda")
    step = max(1, GEN_CHUNK_ELEMS // cols)
    dist = w["dist"]
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        n = (r1 - r0) * cols
        if dist == "normal1":
            x = rng.standard_normal(n, dtype=np.float32)
        elif dist == "normal":
            x = rng.standard_normal(n, dtype=np.float32) * np.float32(0.02)
        elif dist == "normal_outliers":
            x = rng.standard_normal(n, dtype=np.float32) * np.float32(0.02)
            u = rng.random(n, dtype=np.float32)
            x[u < np.float32(0.001)] *= np.float32(50.0)
        elif dist == "laplace":
            u = rng.random(n, dtype=np.float32) - np.float32(0.5)
            x = np.float32(-0.01) * np.sign(u) * np.log1p(np.float32(-2.0) * np.minimum(np.abs(u), np.float32(0.4999999)))
        elif dist == "normal_t3":
            x = rng.standard_normal(n, dtype=np.float32) * np.float32(0.02)
            m = rng.random(n, dtype=np.float32) < np.float32(0.01)
            x[m] = np.float32(0.02) * rng.standard_t(3, int(m.sum())).astype(np.float32)
        else:
            raise ValueError(dist)
        out[r0:r1] = torch.from_numpy(x.astype(np.float32, copy=False).reshape(r1 - r0, cols)).to("cuda").to(dt)
    return out


class Path:
    """Buffers + launches of one workload (quantize_dynamic, quantize, dequantize)."""

    def __init__(self, torch, w, x):
        from cubek_amd import (ComputeClient, ElemType, QuantLevel, QuantScheme, QuantValue,
                               TensorHandleRef)
        from cubek_amd import dequantize as dq, quantize as qz

        self.torch, self.qz, self.dq = torch, qz, dq
        self.elem = ElemType[w["elem"]]
        from cubek_amd import QuantStore

        level = QuantLevel.Tensor if w["block"] is None else QuantLevel.block([w["block"]])
        native = w.get("store", "U32") == "Native"
        self.scheme = (QuantScheme.default().with_value(QuantValue[w["value"]]).with_level(level)
                       .with_store(QuantStore.Native if native else QuantStore.U32))
        shape = tuple(x.shape)
        self.x = x
        if native:  # one byte per value, or two 4-bit values per byte
            per_byte = 2 if w["value"] == "E2M1" else 1
            self.codes = torch.empty(shape[:-1] + (shape[-1] // per_byte,), dtype=torch.uint8, device="cuda")
        else:
            self.codes = torch.empty(self.scheme.packed_shape(shape), dtype=torch.int32, device="cuda")
        self.scales = torch.empty(self.scheme.scales_shape(shape), dtype=torch.float32, device="cuda")
        self.in_scales = torch.empty(self.scheme.scales_shape(shape), dtype=x.dtype, device="cuda")
        self.y = torch.empty_like(x)
        nbytes = qz.workspace_bytes(self.scheme, x.numel())
        self.ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device="cuda")
        self.ws_bytes = nbytes
        self.client = ComputeClient.current()
        h = TensorHandleRef.from_torch
        self.hx, self.hc, self.hs, self.hy, self.his = h(x), h(self.codes), h(self.scales), h(self.y), h(self.in_scales)

    def quantize_dynamic(self):
        self.qz.launch_dynamic(self.client, self.hx, self.hc, self.hs, self.scheme, self.elem,
                               self.ws.data_ptr(), self.ws_bytes)

    def compute_scales(self):
        self.qz.compute_scales(self.client, self.hx, self.his, self.scheme, self.elem,
                               self.ws.data_ptr(), self.ws_bytes)

    def quantize_given(self):
        self.qz.launch_ref(self.client, self.hx, self.hc, self.his, self.hs, self.scheme, self.elem)

    def dequantize(self):
        self.dq.launch_ref(self.client, self.hc, self.hy, self.hs, self.scheme, self.elem)


def timed_region(torch, fn, launches, warmup=3):
    """Runs `launches` back-to-back calls of fn(i) between two HIP events on the launch
    stream (and a host clock bracketed by synchronize).  Returns (event ms per call,
    wall ms per call).  Timing the region as a whole keeps the ~2.5 us an event pair
    adds around a single launch out of the per-kernel figure."""
    for i in range(warmup):
        fn(i)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    a.record()
    for i in range(launches):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return a.elapsed_time(b) / launches, wall * 1e3 / launches


def kernels_in_step(torch, paths, steps, warmup=3):
    """The step's two launches timed where the metric runs them: `steps` steps (quantize, then the dequantize of the
    same set) with an event before, between and after the two launches of each step, all enqueued first.  Returns
    the mean and median of each kernel's per-launch times in ms.  An event between two launches adds ~2.5 us to
    what it brackets, so these read that much longer than a kernel trace of the same launches."""
    for i in range(warmup):
        paths[i % len(paths)].quantize_dynamic()
        paths[i % len(paths)].dequantize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    torch.cuda.synchronize()
    for i in range(steps):
        p = paths[i % len(paths)]
        ev[i][0].record()
        p.quantize_dynamic()
        ev[i][1].record()
        p.dequantize()
        ev[i][2].record()
    torch.cuda.synchronize()
    out = {}
    for name, k in (("quantize", 0), ("dequantize", 1)):
        v = sorted(e[k].elapsed_time(e[k + 1]) for e in ev)
        out[name] = {"avg_launch_ms": sum(v) / len(v), "median_launch_ms": v[len(v) // 2], "launches": len(v)}
    return out


def timed_median(torch, fn, regions=50, warmup=10, region_us=2000.0):
    """The timing protocol of the per-kernel figures: `warmup` untimed launches, then `regions` (>= 50) regions of
    back-to-back launches, each bracketed by HIP events recorded on the launch stream (all regions are enqueued
    first, one synchronize at the end).  A region holds as many launches as fill about `region_us` microseconds
    (2 .. 256), so that what an event between two launches costs (its own ~2.5 us, and the next launch no longer
    starting while the last one drains) stays a small share of a sample.  Returns the median, mean and
    minimum of the per-launch times of the regions, in ms, and the launches per region."""
    for i in range(warmup):
        fn(i)
    est_us = float("inf")
    for _ in range(3):  # the shortest of three probes: the first one after an idle spell can read several times too long
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(8):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        est_us = min(est_us, max(a.elapsed_time(b) / 8 * 1e3, 0.5))
    per = int(min(256, max(2, -(-region_us // est_us))))
    events = [torch.cuda.Event(enable_timing=True) for _ in range(regions + 1)]
    events[0].record()
    k = 0
    for r in range(regions):
        for _ in range(per):
            fn(k)
            k += 1
        events[r + 1].record()
    torch.cuda.synchronize()
    samples = sorted(events[r].elapsed_time(events[r + 1]) / per for r in range(regions))
    return {"median_ms": samples[len(samples) // 2], "mean_ms": sum(samples) / len(samples), "min_ms": samples[0],
            "regions": regions, "launches_per_region": per}


def graph_region(torch, paths, method, launches=32, replays=5):
    """The launches of timed_region captured once into a HIP graph and replayed: the GPU's time
    per launch without the host's share (a call costs the host ~4 us through the Python mirror,
    which bounds eager launches of a few microseconds).  Median over `replays` replays."""

    def one(client, i):
        p = paths[i % len(paths)]
        saved, p.client = p.client, client
        getattr(p, method)()
        p.client = saved

    return graph_region_of(torch, one, len(paths), launches, replays)


def graph_region_of(torch, one, sets, launches=32, replays=5):
    """graph_region for any launch: one(client, i) enqueues launch i on the client's stream."""
    from cubek_amd import ComputeClient

    def run(n):
        client = ComputeClient.current()  # the stream being captured
        for i in range(n):
            one(client, i)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(sets)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(launches)
    graph.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(replays):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        graph.replay()
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) / launches)
    return sorted(times)[len(times) // 2]


def replicas(torch, w, x, min_footprint=1 << 30, max_sets=8, min_sets=1):
    """Independent buffer sets of one workload, enough of them that a launch never
    finds its operands in the 256 MB Infinity Cache or in L2 from the previous
    launch on the same set (cold, HBM-bound timing).  Set 0 holds the seeded
    input; the others hold copies of it."""
    n_sets = max(min_sets, min(max_sets, -(-min_footprint // algorithmic_bytes(w))))
    paths = [Path(torch, w, x)]
    for _ in range(n_sets - 1):
        paths.append(Path(torch, w, x.clone()))
    return paths


def cpu_threads() -> int:
    """Worker threads for the CPU baseline: every hardware thread this process may use, and never more than the
    16 a one-GPU box of this pool gives a job (its CPU share, whatever the core count of the host shows)."""
    return min(16, len(os.sched_getaffinity(0)))


def cpu_baseline(torch, w, path, budget_s=12.0):
    """CPU restatement of the reference algorithm (the oracle, oracle/cq_oracle.c: scalar C, -O2, one pthread per
    slice of words) on a bounded sample of rows of the same tensor: quantize with given scales + dequantize, the
    reference's two launches.  Best of three runs on all threads, and one thread on a shorter sample."""
    import numpy as np

    from oracle import oracle

    rows, cols = w["shape"]
    threads = cpu_threads()
    elem = path.elem

    def host_rows(nrows):
        xs = path.x[:nrows].contiguous()
        if xs.dtype == torch.float32:
            return xs.cpu().numpy()
        return xs.view(torch.int16).cpu().numpy().view(np.uint16)

    def run(nrows, nthreads=threads):
        xs = host_rows(nrows)
        shape = (nrows, cols)
        scales = oracle.compute_scales(xs, elem, shape, path.scheme)  # not timed: the reference takes scales as input
        t0 = time.perf_counter()
        words, out_scale = oracle.quantize(xs, elem, shape, scales, path.scheme, threads=nthreads)
        oracle.dequantize(words, shape, out_scale, elem, path.scheme, threads=nthreads)
        return time.perf_counter() - t0

    probe_rows = max(threads, min(rows, (1 << 21) // cols))
    run(probe_rows)  # first touch: page in the library, start the threads
    t_probe = run(probe_rows)
    # three runs of the sample inside the budget
    nrows = int(min(rows, max(probe_rows, probe_rows * (budget_s / 3.0) / max(t_probe, 1e-3))))
    nrows = max(threads, nrows // threads * threads)
    times = sorted(run(nrows) for _ in range(3))
    t = times[0]
    sample_bytes = 2 * algorithmic_bytes(dict(w, shape=(nrows, cols)))
    # the same on one thread, on a sample an eighth as long
    rows1 = max(1, nrows // 8)
    t1 = min(run(rows1, 1) for _ in range(2))
    bytes1 = 2 * algorithmic_bytes(dict(w, shape=(rows1, cols)))
    return {
        "value": sample_bytes / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
        "what": "CPU restatement of the reference algorithm (this repository's oracle), not the reference's own "
                "CPU runtime, which cannot be built here",
        "sample": f"first {nrows} of {rows} rows of the headline tensor ({nrows * cols} elements), "
                  f"quantize with given scales + dequantize, best of 3 runs: {t:.2f} s on {threads} threads "
                  f"(all three: {', '.join(f'{v:.2f}' for v in times)} s)",
        "elements_per_s": nrows * cols / t,
        "one_thread": {"value": round(bytes1 / t1 / 1e9, 3), "unit": "GB/s", "cores": 1,
                       "sample": f"first {rows1} rows, best of 2 runs: {t1:.2f} s"},
    }


def packed_gemv(torch):
    """The consumer side of the packed format: cq_gemv_quantized over 4-bit weights with f32 scales on blocks of
    32 (configuration 3's weight-load path and four other weights), then other codes, blocks and scale types on
    the largest of them; weights rotated through enough sets that no launch finds them in the Infinity Cache.
    HBM roofline on the packed bytes."""
    from cubek_amd import (ComputeClient, ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue,
                           TensorHandleRef, matvec)

    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    types = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
    cases = [(r, c, "Q4S", [32], "f32", "bf16", "u32") for r, c in ((14336, 4096), (4096, 14336), (28672, 8192),
                                                                    (4096, 11008), (8192, 28672))]
    # (the last element: right-hand vectors, 1 unless given)
    cases += [(28672, 8192, "Q4S", [32], "f32", "bf16", "u32", 4), (14336, 4096, "Q4S", [32], "f32", "bf16", "u32", 4),
              (28672, 8192, "E4M3", [128, 128], "f32", "bf16", "native", 4)]
    cases += [(28672, 8192, "Q4S", [128], "f16", "f16", "u32"), (28672, 8192, "Q4S", [64], "bf16", "bf16", "u32"),
              (28672, 8192, "Q8S", [32], "f32", "bf16", "u32"), (28672, 8192, "Q2S", [64], "f32", "bf16", "u32"),
              (28672, 8192, "E4M3", [128, 128], "f32", "bf16", "native"), (28672, 8192, "E2M1", [32], "f32", "bf16", "native")]
    out = []
    for rows, cols, value, block, param, elem, store, *more in cases:
        vectors = more[0] if more else 1
        scheme = (QuantScheme.default().with_value(QuantValue[value]).with_level(QuantLevel.block(block))
                  .with_param(QuantParam[param.upper()]).with_store(QuantStore.Native if store == "native" else QuantStore.U32))
        nq = scheme.num_quants()
        stored = 4 if store == "u32" else 1  # bytes per stored element
        nscales = (rows // block[0]) * (cols // block[1]) if len(block) == 2 else rows * cols // block[0]
        b = rows * cols // nq * stored + nscales * (4 if param == "f32" else 2) + (cols * 2 + rows * 2) * vectors
        sets = max(2, min(16, -(-(1 << 30) // b)))
        if store == "u32":
            ws = [torch.randint(-2**31, 2**31 - 1, (rows, cols // nq), dtype=torch.int32, device="cuda") for _ in range(sets)]
        else:  # finite codes: e4m3 bytes below 0x78, e2m1 pairs of any nibbles
            ws = [torch.randint(0, 0x78 if value == "E4M3" else 256, (rows, cols // nq), dtype=torch.uint8, device="cuda")
                  for _ in range(sets)]
        sshape = (rows // block[0], cols // block[1]) if len(block) == 2 else (rows, cols // block[0])
        ss = [(torch.rand(sshape, dtype=torch.float32, device="cuda") * 0.01 + 0.001).to(types[param]) for _ in range(sets)]
        x = torch.randn((vectors, cols) if vectors > 1 else cols, device="cuda").to(types[elem])
        y = torch.zeros((vectors, rows) if vectors > 1 else rows, device="cuda", dtype=types[elem])
        hw, hs, hx, hy = [h(t) for t in ws], [h(t) for t in ss], h(x), h(y)
        et = ElemType[elem.upper()]
        fn = lambda i: matvec.launch_ref(client, hw[i % sets], hs[i % sets], scheme, hx, hy, et, et)
        ms = sorted(timed_region(torch, fn, 48)[0] for _ in range(3))[1]
        what = f"{value.lower()[:2]} blocks of {block[0]}" if store == "u32" else \
            f"{value.lower()} ({store} store) blocks of {' x '.join(map(str, block))}"
        out.append({"kernel": f"gemv_quantized, {what}, {param} scales, {elem} x and y, weights [{rows}, {cols}]" +
                              (f", {vectors} right-hand vectors at once" if vectors > 1 else ""),
                    "algorithmic_bytes": b, "buffer_sets_rotated": sets, "ms": round(ms, 4),
                    "GBps": round(b / (ms * 1e-3) / 1e9, 1), "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "weights_per_s": round(rows * cols / (ms * 1e-3)),
                    "multiply_adds_per_s": round(rows * cols * vectors / (ms * 1e-3))})
        rs = read_stream_ms(torch, b)
        if rs is not None:  # the same number of bytes as one plain read stream that computes nothing
            out[-1]["read_stream_same_bytes_ms"] = round(rs, 4)
            out[-1]["frac_of_read_stream"] = round(rs / ms, 4)
        if ms < 0.016:  # within four host enqueue times: also as a replayed HIP graph
            one = lambda c, i: matvec.launch_ref(c, hw[i % sets], hs[i % sets], scheme, hx, hy, et, et)
            g_ms = graph_region_of(torch, one, sets)
            out[-1]["graph_replay_ms"] = round(g_ms, 4)
            out[-1]["graph_replay_frac_hbm_peak"] = round(b / (g_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)
        del ws, ss, hw, hs
    return out


def copy_yardstick(torch, x, launches=24):
    """A plain device-to-device copy of the input tensor (torch.Tensor.copy_, the runtime's copy kernel), timed like
    the kernels of the path on rotated buffers: what this GPU gives a kernel that reads and writes the same
    number of bytes and computes nothing."""
    sets = max(2, min(8, -(-(1 << 30) // (2 * x.numel() * x.element_size()))))
    src = [x] + [x.clone() for _ in range(sets - 1)]
    dst = [torch.empty_like(x) for _ in range(sets)]
    ms = sorted(timed_region(torch, lambda i: dst[i % sets].copy_(src[i % sets]), launches)[0] for _ in range(3))[1]
    b = 2 * x.numel() * x.element_size()
    return {"what": "torch.Tensor.copy_ of the input tensor, device to device, rotated buffer sets",
            "bytes_read_plus_written": b, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
            "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}


PROBES_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cubek_amd", "lib", "libcq_bench_probes.so")


def memory_yardsticks(torch, nbytes, q_read, q_written):
    """What this GPU's memory gives kernels that compute nothing, launched like the streaming kernels (bench probes,
    cubek_amd/csrc/cq_bench_probes.hip): a pure read stream, a pure write stream and a copy of `nbytes`, rotated buffers,
    median of 50 regions.  `additive_ms_*`: the time the headline kernels' own bytes would take as a pure read stream
    plus a pure write stream, which is where reads and writes that do not overlap end up."""
    import ctypes

    if not os.path.exists(PROBES_PATH):
        return {"skipped": f"{PROBES_PATH} is not built (make -C cubek_amd/csrc)"}
    L = ctypes.CDLL(PROBES_PATH)
    L.cq_probe_run.restype = ctypes.c_int
    L.cq_probe_run.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64,
                               ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64)]
    sets = max(4, min(8, -(-(1 << 30) // nbytes)))
    bufs = [torch.randint(0, 2 ** 31 - 1, (nbytes // 4,), dtype=torch.int32, device="cuda") for _ in range(sets)]
    outs = [torch.empty((nbytes // 4,), dtype=torch.int32, device="cuda") for _ in range(sets)]
    stream = torch.cuda.current_stream().cuda_stream
    moved = ctypes.c_uint64(0)
    out = {"what": "read / write / copy kernels that compute nothing (cq_bench_probes.hip), same launch shape as the "
                   "streaming kernels, rotated buffers, median of 50 regions", "bytes": nbytes}
    rates = {}
    for kind, name in ((0, "read_only"), (1, "write_only"), (2, "copy")):
        def fn(i, kind=kind):
            rc = L.cq_probe_run(kind, stream, bufs[i % sets].data_ptr(), outs[i % sets].data_ptr(), nbytes, None,
                                ctypes.byref(moved))
            assert rc == 0, rc
        ms = timed_median(torch, fn)["median_ms"]
        b = moved.value * (2 if kind == 2 else 1)
        rates[name] = moved.value / (ms * 1e-3) / 1e9  # per direction
        out[name] = {"ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                     "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
    out["additive_ms_quantize"] = round((q_read / rates["read_only"] + q_written / rates["write_only"]) * 1e-6, 4)
    out["additive_ms_dequantize"] = round((q_written / rates["read_only"] + q_read / rates["write_only"]) * 1e-6, 4)
    return out


def same_traffic_probes(torch, w):
    """Launches with the traffic of configuration `w`'s quantize and dequantize and none of the arithmetic
    (cq_bench_probes.hip: a workgroup reads 1024 16-byte chunks of floats and writes the share of them that codes and
    scales take, or the reverse; streaming stores), rotated buffers, median of 50 regions: what a kernel of this shape
    that computes nothing takes on this GPU at this size."""
    import ctypes

    if not os.path.exists(PROBES_PATH):
        return None
    L = ctypes.CDLL(PROBES_PATH)
    if not hasattr(L, "cq_probe_shape"):
        return None
    L.cq_probe_shape.restype = ctypes.c_int
    L.cq_probe_shape.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64,
                                 ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64)]
    rows, cols = w["shape"]
    wide = rows * cols * (4 if w["elem"] == "F32" else 2)
    narrow_chunks = max(1, round((algorithmic_bytes(w) - wide) * 1024 / wide))  # of every 1024 chunks of floats
    tiles = wide // 16384
    if tiles == 0:
        return None
    narrow = tiles * narrow_chunks * 16
    sets = max(4, min(16, -(-(1 << 30) // (wide + narrow))))
    wides = [torch.randint(0, 2 ** 31 - 1, (wide // 4,), dtype=torch.int32, device="cuda") for _ in range(sets)]
    narrows = [torch.randint(0, 2 ** 31 - 1, (narrow // 4,), dtype=torch.int32, device="cuda") for _ in range(sets)]
    stream = torch.cuda.current_stream().cuda_stream
    mw, mn = ctypes.c_uint64(0), ctypes.c_uint64(0)
    out = {"narrow_chunks_per_1024": narrow_chunks}
    for widen, name in ((0, "quantize_shaped_ms"), (1, "dequantize_shaped_ms")):
        def fn(i, widen=widen):
            rc = L.cq_probe_shape(widen, stream, wides[i % sets].data_ptr(), narrows[i % sets].data_ptr(), wide,
                                  narrow_chunks, ctypes.byref(mw), ctypes.byref(mn))
            assert rc == 0, rc
        out[name] = round(timed_median(torch, fn)["median_ms"], 4)
    out["bytes_per_launch"] = mw.value + mn.value
    return out


def read_stream_ms(torch, nbytes):
    """A pure read stream of `nbytes` (probe_read_kernel of cq_bench_probes.hip: 16 KiB per workgroup, consecutive
    lanes on consecutive 16 bytes), rotated buffers of at least 1 GiB together, median of 50 regions."""
    import ctypes

    if not os.path.exists(PROBES_PATH):
        return None
    L = ctypes.CDLL(PROBES_PATH)
    L.cq_probe_run.restype = ctypes.c_int
    L.cq_probe_run.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64,
                               ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64)]
    nbytes = nbytes // 16384 * 16384
    if nbytes == 0:
        return None
    sets = max(4, min(32, -(-(1 << 30) // nbytes)))
    bufs = [torch.randint(0, 2 ** 31 - 1, (nbytes // 4,), dtype=torch.int32, device="cuda") for _ in range(sets)]
    stream = torch.cuda.current_stream().cuda_stream

    def fn(i):
        rc = L.cq_probe_run(0, stream, bufs[i % sets].data_ptr(), None, nbytes, None, None)
        assert rc == 0, rc
    return timed_median(torch, fn)["median_ms"]


def transposed_tile_probes(torch, widen, floats, codes, scales, rows, cols):
    """The traffic of the transposed tile kernels without their arithmetic (cq_probe_transposed in cq_bench_probes.hip:
    tiles of 128 rows x 256 columns, 256-byte runs of floats on one side, 128 bytes of codes and 32 of scales per row
    on the other), on the buffers of the rows they stand beside: streaming or ordinary stores, tiles in launch order
    or XCD by XCD; medians of 50 regions each and the best of the four."""
    import ctypes

    if not os.path.exists(PROBES_PATH):
        return None
    L = ctypes.CDLL(PROBES_PATH)
    if not hasattr(L, "cq_probe_transposed"):
        return None
    L.cq_probe_transposed.restype = ctypes.c_int
    L.cq_probe_transposed.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32]
    if rows % 128 or cols % 256:
        return None
    assert all(t.numel() * t.element_size() >= rows * cols * 2 for t in floats)
    assert all(t.numel() * t.element_size() >= rows * cols // 2 for t in codes)
    assert all(t.numel() * t.element_size() >= rows * cols // 8 for t in scales)
    stream = torch.cuda.current_stream().cuda_stream
    # (widen: the probe overwrites `floats`; the caller passes output buffers)
    out = {}
    for plain in (0, 1):
        for xcd in (0, 1):
            def fn(i, plain=plain, xcd=xcd):
                rc = L.cq_probe_transposed(int(widen), plain, xcd, stream, floats[i % len(floats)].data_ptr(),
                                           codes[i % len(codes)].data_ptr(), scales[i % len(scales)].data_ptr(), rows, cols)
                assert rc == 0, rc
            name = ("ordinary" if plain else "streaming") + " stores, " + ("tiles XCD by XCD" if xcd else "tiles in launch order")
            out[name] = round(timed_median(torch, fn)["median_ms"], 4)
    return {"variants_ms": out, "best_ms": min(out.values())}


def scheme_matrix(torch):
    """Every float type x value x store on the headline shape, blocks of 32, f32 parameters: the three launches of
    the path, reported only (`--matrix`).  Inputs ~N(0, 0.02) from torch's generator, three rotated buffer sets."""
    rows, cols = WORKLOADS["cfg5"]["shape"]
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    base = torch.randn((rows, cols), generator=g, device="cuda", dtype=torch.float32).mul_(0.02)
    out = []
    for elem, tdt in (("BF16", torch.bfloat16), ("F16", torch.float16), ("F32", torch.float32)):
        x = base.to(tdt)
        for value, store, bits in (("Q8S", "U32", 8), ("Q4S", "U32", 4), ("Q2S", "U32", 2), ("E2M1", "U32", 4),
                                   ("Q8S", "Native", 8), ("E4M3", "Native", 8),
                                   ("E5M2", "Native", 8), ("E2M1", "Native", 4)):
            w = dict(shape=(rows, cols), elem=elem, value=value, block=32, store=store)
            ps = [Path(torch, w, x if i == 0 else x.clone()) for i in range(3)]
            b = rows * cols * x.element_size() + rows * cols * bits // 8 + rows * cols // 32 * 4
            for p in ps:
                p.compute_scales()
            row = {"elem": elem, "value": value, "store": store, "algorithmic_bytes": b}
            for label, meth in (("quantize_dynamic", "quantize_dynamic"), ("quantize_given_scales", "quantize_given"),
                                ("dequantize", "dequantize")):
                fn = lambda i, m=meth: getattr(ps[i % len(ps)], m)()
                ms = sorted(timed_region(torch, fn, 16)[0] for _ in range(3))[1]
                row[label] = {"ms": round(ms, 4), "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
            out.append(row)
            del ps, p
        del x
    return out


def adjacent_kernels(torch):
    """The steps either side of the path on the headline tensor: abs-max along an axis
    (cq_reduce_max_abs) in front of it, 2-D blocks, a transposed float tensor, pitched rows and an
    attention layout through the path itself, re-packing of a transposed quantized tensor (cq_into_contiguous_packed)
    behind it.  Reported only; `value` does not include them."""
    from cubek_amd import ComputeClient, ElemType, TensorHandleRef
    from cubek_amd import contiguous as cq_contiguous
    from cubek_amd import reduce as cq_reduce

    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    rows, cols = WORKLOADS["cfg5"]["shape"]
    sets = 4  # 4 x 470 MB: each launch reads a tensor that has left the Infinity Cache
    xs = [torch.randn((rows, cols), device="cuda", dtype=torch.bfloat16) for _ in range(sets)]
    out = []
    for axis in (1, 0):
        o = torch.zeros((rows, 1) if axis == 1 else (1, cols), device="cuda", dtype=torch.bfloat16)
        nbytes = cq_reduce.workspace_bytes(h(xs[0]), axis, ElemType.BF16)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
        hs, ho = [h(x) for x in xs], h(o)
        fn = lambda i: cq_reduce.max_abs(client, hs[i % sets], ho, axis, ElemType.BF16, ws.data_ptr() if nbytes else 0,
                                         nbytes)
        ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
        b = rows * cols * 2
        out.append({"kernel": f"reduce_max_abs axis {axis} of bf16 [{rows}, {cols}]", "algorithmic_bytes": b,
                    "workspace_bytes": nbytes, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
    # the same buffers seen transposed ([cols, rows] with strides (1, cols)): reduced in the order of their strides
    for axis in (0, 1):
        o = torch.zeros((1, rows) if axis == 0 else (cols, 1), device="cuda", dtype=torch.bfloat16)
        hs = [TensorHandleRef(h(x).handle, (cols, rows), (1, cols), 2) for x in xs]
        nbytes = cq_reduce.workspace_bytes(hs[0], axis, ElemType.BF16)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
        ho = h(o)
        fn = lambda i: cq_reduce.max_abs(client, hs[i % sets], ho, axis, ElemType.BF16, ws.data_ptr() if nbytes else 0,
                                         nbytes)
        ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
        b = rows * cols * 2
        out.append({"kernel": f"reduce_max_abs axis {axis} of the transposed bf16 view [{cols}, {rows}]", "algorithmic_bytes": b,
                    "workspace_bytes": nbytes, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
    # weight-style 128 x 128 blocks, fp8 e4m3 bytes: the fused block kernel (one launch, one read)
    from cubek_amd import QuantLevel, QuantScheme, QuantStore, QuantValue
    from cubek_amd import dequantize as cq_dequantize
    from cubek_amd import quantize as cq_quantize

    scheme = (QuantScheme.default().with_value(QuantValue.E4M3).with_store(QuantStore.Native)
              .with_level(QuantLevel.block([128, 128])))
    codes = [torch.empty((rows, cols), dtype=torch.uint8, device="cuda") for _ in range(sets)]
    scales = [torch.empty((rows // 128, cols // 128), dtype=torch.float32, device="cuda") for _ in range(sets)]
    ys = [torch.empty((rows, cols), dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    hx, hc, hs, hy = [h(x) for x in xs], [h(c) for c in codes], [h(s) for s in scales], [h(y) for y in ys]
    b = rows * cols * 3 + scales[0].numel() * 4
    for label, fn in (
            ("quantize_dynamic", lambda i: cq_quantize.launch_dynamic(client, hx[i % sets], hc[i % sets], hs[i % sets],
                                                                       scheme, ElemType.BF16)),
            ("dequantize", lambda i: cq_dequantize.launch_ref(client, hc[i % sets], hy[i % 2], hs[i % sets], scheme,
                                                              ElemType.BF16))):
        ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
        out.append({"kernel": f"{label}, 128 x 128 blocks, e4m3 native store, bf16 [{rows}, {cols}]",
                    "algorithmic_bytes": b, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
    # the headline scheme on a transposed float tensor: a [cols, rows] buffer viewed as [rows, cols]
    scheme = QuantScheme.default().with_value(QuantValue.E2M1).with_level(QuantLevel.block([32]))
    words = [torch.empty((rows, cols // 8), dtype=torch.int32, device="cuda") for _ in range(2)]
    bscales = [torch.empty((rows, cols // 32), dtype=torch.float32, device="cuda") for _ in range(2)]
    transposed = lambda t: TensorHandleRef(h(t).handle, (rows, cols), (1, rows), 2)
    hxt = [transposed(x.view(cols, rows)) for x in xs]
    hyt = [transposed(y.view(cols, rows)) for y in ys]
    hw, hb = [h(t) for t in words], [h(t) for t in bscales]
    b = rows * cols * 2 + rows * cols // 2 + bscales[0].numel() * 4
    for label, fn in (
            ("quantize_dynamic", lambda i: cq_quantize.launch_dynamic(client, hxt[i % sets], hw[i % 2], hb[i % 2], scheme,
                                                                       ElemType.BF16)),
            ("dequantize", lambda i: cq_dequantize.launch_ref(client, hw[i % 2], hyt[i % 2], hb[i % 2], scheme,
                                                              ElemType.BF16))):
        ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
        out.append({"kernel": f"{label}, e2m1 blocks of 32, transposed bf16 view [{rows}, {cols}] of a [{cols}, {rows}] buffer",
                    "algorithmic_bytes": b, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        probe = transposed_tile_probes(torch, label == "dequantize", ys if label == "dequantize" else xs, words, bscales, rows, cols)
        if probe is not None:
            out[-1]["same_traffic_no_arithmetic"] = probe
            out[-1]["frac_of_same_traffic_probe"] = round(probe["best_ms"] / ms, 4)
    # one scale per tensor: two launches, the tensor read twice (pass 1 leaves what it can in the caches for pass 2)
    tensor_scheme = QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.Tensor)
    ws_bytes = cq_quantize.workspace_bytes(tensor_scheme, rows * cols)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device="cuda")
    for pr, pc in ((rows, cols), (8192, 8192), (4096, 4096)):
        n_sets = sets if (pr, pc) == (rows, cols) else 8
        xq = xs if (pr, pc) == (rows, cols) else [torch.randn((pr, pc), device="cuda", dtype=torch.bfloat16) for _ in range(n_sets)]
        words = [torch.empty((pr, pc // 4), dtype=torch.int32, device="cuda") for _ in range(2)]
        one = [torch.empty((1,), dtype=torch.float32, device="cuda") for _ in range(2)]
        hxq, hw, ho = [h(t) for t in xq], [h(t) for t in words], [h(t) for t in one]
        fn = lambda i: cq_quantize.launch_dynamic(client, hxq[i % n_sets], hw[i % 2], ho[i % 2], tensor_scheme, ElemType.BF16,
                                                  ws.data_ptr(), ws_bytes)
        ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
        b = pr * pc * 3 + 4
        out.append({"kernel": f"quantize_dynamic, q8 per tensor (two passes), bf16 [{pr}, {pc}]", "algorithmic_bytes": b,
                    "buffer_sets_rotated": n_sets, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        del xq, words, one, hxq, hw, ho
    del xs, codes, scales, ys, hx, hc, hs, hy, bscales, hxt, hyt, hb
    # the headline scheme on pitched rows: [rows, cols] views of [rows, cols + 64] buffers, at the headline
    # row length and with the same elements in rows a quarter as long
    # ... with rows whose last step of 256 chunks is cut short (576 chunks a row), and with bf16 parameters on the
    # contiguous tensor: the layouts that the lane-wise streaming kernels take whole
    from cubek_amd import QuantParam

    f32_scheme = scheme
    for pr, pc, pad, param in ((rows, cols, 64, "F32"), (rows * 4, cols // 4, 64, "F32"), (32768, 4608, 64, "F32"),
                               (rows, cols, 0, "BF16")):
        scheme = f32_scheme.with_param(QuantParam[param])
        xp = [torch.randn((pr, pc + pad), device="cuda", dtype=torch.bfloat16) for _ in range(sets)]
        yp = [torch.empty((pr, pc + pad), device="cuda", dtype=torch.bfloat16) for _ in range(2)]
        words = [torch.empty((pr, pc // 8), dtype=torch.int32, device="cuda") for _ in range(2)]
        bscales = [torch.empty((pr, pc // 32), dtype=torch.float32 if param == "F32" else torch.bfloat16, device="cuda")
                   for _ in range(2)]
        pitched = lambda t: TensorHandleRef(h(t).handle, (pr, pc), (pc + pad, 1), 2)
        hxp, hyp = [pitched(t) for t in xp], [pitched(t) for t in yp]
        hw, hb = [h(t) for t in words], [h(t) for t in bscales]
        b = pr * pc * 2 + pr * pc // 2 + bscales[0].numel() * bscales[0].element_size()
        what = (f"pitched bf16 rows: [{pr}, {pc}] view of a [{pr}, {pc + pad}] buffer" if pad else
                f"contiguous bf16 [{pr}, {pc}]") + ("" if param == "F32" else f", {param.lower()} parameters")
        for label, fn in (
                ("quantize_dynamic", lambda i: cq_quantize.launch_dynamic(client, hxp[i % sets], hw[i % 2], hb[i % 2], scheme,
                                                                           ElemType.BF16)),
                ("dequantize", lambda i: cq_dequantize.launch_ref(client, hw[i % 2], hyp[i % 2], hb[i % 2], scheme,
                                                                  ElemType.BF16))):
            ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
            out.append({"kernel": f"{label}, e2m1 blocks of 32, {what}",
                        "algorithmic_bytes": b, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                        "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        if pc == cols and pad:  # abs-max along both axes of the same pitched rows
            for axis in (1, 0):
                o = torch.zeros((pr, 1) if axis == 1 else (1, pc), device="cuda", dtype=torch.bfloat16)
                nbytes = cq_reduce.workspace_bytes(hxp[0], axis, ElemType.BF16)
                ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
                ho = h(o)
                fn = lambda i: cq_reduce.max_abs(client, hxp[i % sets], ho, axis, ElemType.BF16,
                                                 ws.data_ptr() if nbytes else 0, nbytes)
                ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
                out.append({"kernel": f"reduce_max_abs axis {axis} of pitched bf16 rows: [{pr}, {pc}] view of a [{pr}, {pc + pad}] buffer",
                            "algorithmic_bytes": pr * pc * 2, "workspace_bytes": nbytes, "ms": round(ms, 4),
                            "GBps": round(pr * pc * 2 / (ms * 1e-3) / 1e9, 1),
                            "frac_hbm_peak": round(pr * pc * 2 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        del xp, yp, words, bscales, hxp, hyp, hw, hb
    scheme = f32_scheme
    # the headline scheme on an attention layout: the [batch, heads, positions, head dimension] view of a
    # [batch, positions, heads, head dimension] buffer (rows of 128 elements behind permuted dimensions)
    nb, nh, ns, nd = 8, 32, 4096, 128
    xa = [torch.randn((nb, ns, nh, nd), device="cuda", dtype=torch.bfloat16) for _ in range(sets)]
    ya = [torch.empty((nb, ns, nh, nd), device="cuda", dtype=torch.bfloat16) for _ in range(2)]
    # four output sets as well: two (168 MB) would stay in the 256 MB Infinity Cache and never reach HBM
    words = [torch.empty((nb, nh, ns, nd // 8), dtype=torch.int32, device="cuda") for _ in range(sets)]
    bscales = [torch.empty((nb, nh, ns, nd // 32), dtype=torch.float32, device="cuda") for _ in range(sets)]
    heads = lambda t: TensorHandleRef(h(t).handle, (nb, nh, ns, nd), (ns * nh * nd, nd, nh * nd, 1), 2)
    hxa, hya = [heads(t) for t in xa], [heads(t) for t in ya]
    hw, hb = [h(t) for t in words], [h(t) for t in bscales]
    b = nb * nh * ns * nd * 2 + words[0].numel() * 4 + bscales[0].numel() * 4
    for label, fn in (
            ("quantize_dynamic", lambda i: cq_quantize.launch_dynamic(client, hxa[i % sets], hw[i % sets], hb[i % sets], scheme,
                                                                       ElemType.BF16)),
            ("dequantize", lambda i: cq_dequantize.launch_ref(client, hw[i % sets], hya[i % 2], hb[i % sets], scheme,
                                                              ElemType.BF16))):
        ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
        out.append({"kernel": f"{label}, e2m1 blocks of 32, bf16 [{nb}, {nh}, {ns}, {nd}] view of a [{nb}, {ns}, {nh}, {nd}] buffer",
                    "algorithmic_bytes": b, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
    del xa, ya, words, bscales, hxa, hya, hw, hb
    # the kernels that stage through LDS: blocks that are not a power of two of 16-byte chunks (24 values of 4 bits),
    # and the headline scheme with its scales stored column by column (given scales: read row by row, out_scale
    # written column by column)
    for pr, pc, value, block, col_major in ((rows, cols - 8, "Q4S", 24, False), (rows, cols, "E2M1", 32, True)):
        rscheme = QuantScheme.default().with_value(QuantValue[value]).with_level(QuantLevel.block([block]))
        nbk = pc // block
        xr = [torch.randn((pr, pc), device="cuda", dtype=torch.bfloat16) for _ in range(sets)]
        yr = [torch.empty((pr, pc), device="cuda", dtype=torch.bfloat16) for _ in range(2)]
        wr = [torch.empty((pr, pc // 8), dtype=torch.int32, device="cuda") for _ in range(sets)]
        given = [torch.rand((pr, nbk), device="cuda").mul_(0.01).add_(0.01).to(torch.bfloat16) for _ in range(sets)]
        if col_major:
            sr = [torch.rand((nbk, pr), device="cuda").mul_(0.01).add_(0.01) for _ in range(sets)]
            hsr = [TensorHandleRef(h(t).handle, (pr, nbk), (1, pr), 4) for t in sr]
        else:
            sr = [torch.rand((pr, nbk), device="cuda").mul_(0.01).add_(0.01) for _ in range(sets)]
            hsr = [h(t) for t in sr]
        hxr, hyr, hwr, hgr = [h(t) for t in xr], [h(t) for t in yr], [h(t) for t in wr], [h(t) for t in given]
        b = pr * pc * 2 + wr[0].numel() * 4 + sr[0].numel() * 4
        what = f"{value.lower()} blocks of {block}, bf16 [{pr}, {pc}]" + (", scales stored column by column" if col_major else "")
        calls = [("quantize (given scales)", lambda i: cq_quantize.launch_ref(client, hxr[i % sets], hwr[i % sets], hgr[i % sets],
                                                                             hsr[i % sets], rscheme, ElemType.BF16)),
                 ("dequantize", lambda i: cq_dequantize.launch_ref(client, hwr[i % sets], hyr[i % 2], hsr[i % sets], rscheme,
                                                                   ElemType.BF16))]
        calls.insert(1, ("quantize_dynamic", lambda i: cq_quantize.launch_dynamic(client, hxr[i % sets], hwr[i % sets],
                                                                                  hsr[i % sets], rscheme, ElemType.BF16)))
        for label, fn in calls:
            ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
            out.append({"kernel": f"{label}, {what}", "algorithmic_bytes": b, "ms": round(ms, 4),
                        "GBps": round(b / (ms * 1e-3) / 1e9, 1), "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        del xr, yr, wr, given, sr, hsr, hxr, hyr, hwr, hgr
    # 4-bit codes of a [rows, cols] weight, 8 per u32 word along cols, viewed transposed as [cols, rows]
    packing = 8
    srcs = [torch.randint(-2**31, 2**31 - 1, (rows, cols // packing), dtype=torch.int32, device="cuda")
            for _ in range(8)]
    dst = torch.zeros((cols, rows // packing), dtype=torch.int32, device="cuda")
    hs = [TensorHandleRef(h(t).handle, (cols // packing, rows), (1, cols // packing), 4) for t in srcs]
    hd = h(dst)
    fn = lambda i: cq_contiguous.into_contiguous_packed_ref(client, hs[i % len(hs)], hd, (cols, rows), packing)
    ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
    b = 2 * rows * cols // packing * 4
    out.append({"kernel": f"into_contiguous_packed of transposed 4-bit [{cols}, {rows}] (u32 x 8)",
                "algorithmic_bytes": b, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
    # the same codes with pitched rows ([rows, cols/8 - 8] words out of every row of cols/8): a copy of strided rows
    wcols = cols // packing - 8
    hs = [TensorHandleRef(h(t).handle, (rows, wcols), (cols // packing, 1), 4) for t in srcs]
    hd = TensorHandleRef(h(dst).handle, (rows, wcols), (wcols, 1), 4)
    fn = lambda i: cq_contiguous.into_contiguous_packed_ref(client, hs[i % len(hs)], hd, (rows, wcols * packing), packing)
    ms = sorted(timed_region(torch, fn, 24)[0] for _ in range(3))[1]
    b = 2 * rows * wcols * 4
    out.append({"kernel": f"into_contiguous_packed of 4-bit rows with a pitch: [{rows}, {wcols}] words out of [{rows}, {cols // packing}]",
                "algorithmic_bytes": b, "ms": round(ms, 4), "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
    return out


def corner_layouts(torch):
    """Layouts that ran one thread per stored element before they had kernels of their own, on the headline tensor's
    size: rows that start on odd multiples of 2 bytes, a stored tensor whose last dimension is not the contiguous one,
    E4M3 in the u32 store (codes that wrap their field), and an abs-max whose output is strided."""
    from cubek_amd import ComputeClient, ElemType, QuantLevel, QuantScheme, QuantValue, TensorHandleRef, _ffi
    from cubek_amd import dequantize as cq_dequantize
    from cubek_amd import quantize as cq_quantize
    from cubek_amd import reduce as cq_reduce

    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    rows, cols = WORKLOADS["cfg5"]["shape"]
    sets = 4
    out = []

    def record(label, b, fn, family):
        ms = sorted(timed_region(torch, fn, 12, warmup=2)[0] for _ in range(3))[1]
        out.append({"kernel": label, "family": family, "algorithmic_bytes": b, "ms": round(ms, 4),
                    "GBps": round(b / (ms * 1e-3) / 1e9, 1), "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})

    scheme = QuantScheme.default().with_value(QuantValue.E2M1).with_level(QuantLevel.block([32]))
    words = [torch.empty((rows, cols // 8), dtype=torch.int32, device="cuda") for _ in range(sets)]
    scales = [torch.empty((rows, cols // 32), dtype=torch.float32, device="cuda") for _ in range(sets)]
    hw, hs = [h(t) for t in words], [h(t) for t in scales]
    b = rows * cols * 2 + rows * cols // 2 + rows * cols // 32 * 4
    # 1. rows of cols + 1 elements: every other row starts on an odd multiple of 2 bytes
    xo = [torch.randn((rows, cols + 1), device="cuda", dtype=torch.bfloat16) for _ in range(sets)]
    yo = [torch.empty((rows, cols + 1), device="cuda", dtype=torch.bfloat16) for _ in range(2)]
    odd = lambda t: TensorHandleRef(h(t).handle, (rows, cols), (cols + 1, 1), 2)
    hxo, hyo = [odd(t) for t in xo], [odd(t) for t in yo]
    fam = _ffi.plan_kind(_ffi.OP_QUANTIZE_DYNAMIC, hxo[0], hw[0], None, hs[0], scheme, ElemType.BF16)
    record(f"quantize_dynamic, e2m1 blocks of 32, bf16 rows [{rows}, {cols}] with a pitch of {cols + 1} elements", b,
           lambda i: cq_quantize.launch_dynamic(client, hxo[i % sets], hw[i % sets], hs[i % sets], scheme, ElemType.BF16), fam)
    fam = _ffi.plan_kind(_ffi.OP_DEQUANTIZE, hyo[0], hw[0], hs[0], None, scheme, ElemType.BF16)
    record(f"dequantize, e2m1 blocks of 32, bf16 rows [{rows}, {cols}] with a pitch of {cols + 1} elements", b,
           lambda i: cq_dequantize.launch_ref(client, hw[i % sets], hyo[i % 2], hs[i % sets], scheme, ElemType.BF16), fam)
    del xo, yo, hxo, hyo
    # 2. the stored tensor transposed in memory: word (r, w) at w * rows + r
    xs = [torch.randn((rows, cols), device="cuda", dtype=torch.bfloat16) for _ in range(sets)]
    ys = [torch.empty((rows, cols), device="cuda", dtype=torch.bfloat16) for _ in range(2)]
    hx, hy = [h(t) for t in xs], [h(t) for t in ys]
    hwt = [TensorHandleRef(h(t).handle, (rows, cols // 8), (1, rows), 4) for t in words]
    fam = _ffi.plan_kind(_ffi.OP_QUANTIZE_DYNAMIC, hx[0], hwt[0], None, hs[0], scheme, ElemType.BF16)
    record(f"quantize_dynamic, e2m1 blocks of 32, bf16 [{rows}, {cols}], stored tensor with strides (1, {rows})", b,
           lambda i: cq_quantize.launch_dynamic(client, hx[i % sets], hwt[i % sets], hs[i % sets], scheme, ElemType.BF16), fam)
    fam = _ffi.plan_kind(_ffi.OP_DEQUANTIZE, hy[0], hwt[0], hs[0], None, scheme, ElemType.BF16)
    record(f"dequantize, e2m1 blocks of 32, bf16 [{rows}, {cols}], stored tensor with strides (1, {rows})", b,
           lambda i: cq_dequantize.launch_ref(client, hwt[i % sets], hy[i % 2], hs[i % sets], scheme, ElemType.BF16), fam)
    # 3. E4M3 in the u32 store
    e4 = QuantScheme.default().with_value(QuantValue.E4M3).with_level(QuantLevel.block([32]))
    w8 = [torch.empty((rows, cols // 4), dtype=torch.int32, device="cuda") for _ in range(sets)]
    hw8 = [h(t) for t in w8]
    b8 = rows * cols * 2 + rows * cols + rows * cols // 32 * 4
    fam = _ffi.plan_kind(_ffi.OP_QUANTIZE_DYNAMIC, hx[0], hw8[0], None, hs[0], e4, ElemType.BF16)
    record(f"quantize_dynamic, e4m3 in the u32 store (fields wrap), blocks of 32, bf16 [{rows}, {cols}]", b8,
           lambda i: cq_quantize.launch_dynamic(client, hx[i % sets], hw8[i % sets], hs[i % sets], e4, ElemType.BF16), fam)
    del w8, hw8
    # 3b. the extension value E2M1_OCP (e2m1 nibbles rounded once from the quotient; not a scheme of the reference) in the
    # u32 store, contiguous: the headline kernels with the e2m1 conversion instead of the integer packing
    oc = QuantScheme.default().with_value(QuantValue.E2M1_OCP).with_level(QuantLevel.block([32]))
    fam = _ffi.plan_kind(_ffi.OP_QUANTIZE_DYNAMIC, hx[0], hw[0], None, hs[0], oc, ElemType.BF16)
    record(f"quantize_dynamic, e2m1_ocp (extension) blocks of 32, u32 store, bf16 [{rows}, {cols}]", b,
           lambda i: cq_quantize.launch_dynamic(client, hx[i % sets], hw[i % sets], hs[i % sets], oc, ElemType.BF16), fam)
    fam = _ffi.plan_kind(_ffi.OP_DEQUANTIZE, hy[0], hw[0], hs[0], None, oc, ElemType.BF16)
    record(f"dequantize, e2m1_ocp (extension) blocks of 32, u32 store, bf16 [{rows}, {cols}]", b,
           lambda i: cq_dequantize.launch_ref(client, hw[i % sets], hy[i % 2], hs[i % sets], oc, ElemType.BF16), fam)
    # 4. abs-max along the rows into column 1 of a [rows, 4] tensor, and along the columns into every other element
    for axis, oshape, ostr in ((1, (rows, 1), (4, 1)), (0, (1, cols), (2 * cols, 2))):
        o = torch.zeros(rows * 4 if axis == 1 else cols * 2, device="cuda", dtype=torch.bfloat16)
        ho = TensorHandleRef(o.data_ptr() + (2 if axis == 1 else 0), oshape, ostr, 2)
        nbytes = cq_reduce.workspace_bytes(hx[0], axis, ElemType.BF16)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
        record(f"reduce_max_abs axis {axis} of bf16 [{rows}, {cols}] into an output with strides {ostr}", rows * cols * 2,
               lambda i: cq_reduce.max_abs(client, hx[i % sets], ho, axis, ElemType.BF16, ws.data_ptr() if nbytes else 0, nbytes),
               "-")
    return out


def per_tensor_passes(torch):
    """Where the time of a per-tensor dynamic quantize goes, at sizes that fit the 256 MB Infinity Cache: the two
    passes timed apart through the public entry points (cq_compute_scales = pass 1 + the scale; cq_quantize with that
    scale = what pass 2 does), the second one on a tensor that has left the caches (eight rotated inputs) and right
    behind pass 1 on the same tensor, and cq_quantize_dynamic itself.  q8 of bf16."""
    from cubek_amd import ComputeClient, ElemType, QuantLevel, QuantScheme, QuantValue, TensorHandleRef
    from cubek_amd import quantize as cq_quantize

    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    scheme = QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.Tensor)
    out = []
    for rows, cols in ((4096, 4096), (8192, 4096), (8192, 8192)):
        sets = 8
        xs = [torch.randn((rows, cols), device="cuda", dtype=torch.bfloat16) for _ in range(sets)]
        words = [torch.empty((rows, cols // 4), dtype=torch.int32, device="cuda") for _ in range(2)]
        sc_in = [torch.ones((1,), dtype=torch.bfloat16, device="cuda") for _ in range(sets)]
        sc_out = [torch.empty((1,), dtype=torch.float32, device="cuda") for _ in range(2)]
        ws_bytes = cq_quantize.workspace_bytes(scheme, rows * cols)
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device="cuda")
        hx, hw, hsi, hso = [h(t) for t in xs], [h(t) for t in words], [h(t) for t in sc_in], [h(t) for t in sc_out]
        pass1 = lambda i: cq_quantize.compute_scales(client, hx[i % sets], hsi[i % sets], scheme, ElemType.BF16, ws.data_ptr(), ws_bytes)
        pass2 = lambda i: cq_quantize.launch_ref(client, hx[i % sets], hw[i % 2], hsi[i % sets], hso[i % 2], scheme, ElemType.BF16)

        def pair(i):
            pass1(i)
            pass2(i)
        dyn = lambda i: cq_quantize.launch_dynamic(client, hx[i % sets], hw[i % 2], hso[i % 2], scheme, ElemType.BF16,
                                                   ws.data_ptr(), ws_bytes)
        again = lambda i: cq_quantize.compute_scales(client, hx[0], hsi[0], scheme, ElemType.BF16, ws.data_ptr(), ws_bytes)
        t = {k: sorted(timed_region(torch, f, 32)[0] for _ in range(3))[1]
             for k, f in (("pass1", pass1), ("pass1_again", again), ("pass2_cold", pass2), ("pair", pair), ("dynamic", dyn))}
        mib = rows * cols * 2 >> 20
        b = rows * cols * 3 + 4
        out.append({"kernel": f"per-tensor q8 of bf16 [{rows}, {cols}] ({mib} MiB), the two passes apart",
                    "algorithmic_bytes": b, "ms": round(t["dynamic"], 4),
                    "GBps": round(b / (t["dynamic"] * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(b / (t["dynamic"] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "pass1_abs_max_and_scale_ms": round(t["pass1"], 4),
                    "pass1_GBps_on_the_input": round(rows * cols * 2 / (t["pass1"] * 1e-3) / 1e9, 1),
                    # the same launches on ONE tensor, over and over: what a read gains from finding its operand
                    # in the Infinity Cache
                    "pass1_on_the_same_tensor_again_ms": round(t["pass1_again"], 4),
                    "pass2_on_a_cold_tensor_ms": round(t["pass2_cold"], 4),
                    "pass2_behind_pass1_ms": round(t["pair"] - t["pass1"], 4),
                    "both_passes_as_two_calls_ms": round(t["pair"], 4)})
        del xs, words, hx, hw
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg5", choices=sorted(WORKLOADS))
    ap.add_argument("--no-sweep", action="store_true", help="skip the per-config table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--adjacent-only", action="store_true",
                    help="run only the abs-max / re-pack kernels on the headline tensor (for profiling)")
    ap.add_argument("--gemv-only", action="store_true",
                    help="run only the matrix-vector product over packed weights (for profiling)")
    ap.add_argument("--corners-only", action="store_true",
                    help="run only the layouts that used to run one thread per element (for profiling)")
    ap.add_argument("--matrix", action="store_true",
                    help="run only the float type x value x store matrix on the headline shape (reported only)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run 3 plain device copies of the input (known bytes) to calibrate rocprof counters")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU part (per-block quantization "
                 "shards by rows without communication); run with --gpus 1")

    import torch

    from cubek_amd import _ffi

    _ffi.lib()  # fail loudly if the HIP library is not built
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    if args.adjacent_only:
        print(json.dumps({"adjacent_kernels": adjacent_kernels(torch) + corner_layouts(torch) + per_tensor_passes(torch) + packed_gemv(torch)}))
        return
    if args.corners_only:
        print(json.dumps({"adjacent_kernels": corner_layouts(torch) + per_tensor_passes(torch)}))
        return
    if args.gemv_only:
        print(json.dumps({"adjacent_kernels": packed_gemv(torch)}))
        return
    if args.matrix:
        print(json.dumps({"scheme_matrix": scheme_matrix(torch)}))
        return

    w = WORKLOADS[args.workload]
    x = make_input(torch, w)
    q_bytes = algorithmic_bytes(w)
    step_bytes = 2 * q_bytes
    n = x.numel()

    # (at least four sets: with two, a tenth of a set's input is still in the 256 MB Infinity Cache when its turn comes
    # again (the headline quantize launch reads 97 us with two sets, 100.0 - 100.5 us with three to eight); and where
    # the buffers lie in memory moves a launch by up to 2 %, which four placements average)
    paths = replicas(torch, w, x, min_sets=4)
    path = paths[0]
    # the process's first launches: what the runtime takes to load the library's code objects is in here
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    path.quantize_dynamic()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    path.dequantize()
    torch.cuda.synchronize()
    first_ms = [(t1 - t0) * 1e3, (time.perf_counter() - t1) * 1e3]

    def step(i):
        p = paths[i % len(paths)]
        p.quantize_dynamic()
        p.dequantize()

    # The clocks of a GPU that has been idle take a few hundred milliseconds of load to settle (the first regions of a
    # fresh process read 3 - 5 % slower than everything after them): load it for about 0.4 s before anything is timed.
    settle_until = time.perf_counter() + 0.4
    while time.perf_counter() < settle_until:
        for i in range(16):
            step(i)
        torch.cuda.synchronize()
    # timed region: exactly K steps between synchronize() calls
    ev_ms, ms_per_step = timed_region(torch, step, args.steps, warmup=args.warmup)
    # the two kernels of the step, each alone: the average over one region of K back-to-back launches (what a
    # rocprofv3 kernel trace of this command averages), and the median of 50 event-timed regions
    q_ms, _ = timed_region(torch, lambda i: paths[i % len(paths)].quantize_dynamic(), args.steps)
    d_ms, _ = timed_region(torch, lambda i: paths[i % len(paths)].dequantize(), args.steps)
    q_med = timed_median(torch, lambda i: paths[i % len(paths)].quantize_dynamic())
    d_med = timed_median(torch, lambda i: paths[i % len(paths)].dequantize())
    # and the same two launches inside the step, where the quantize launch runs about a tenth shorter than alone
    in_step = kernels_in_step(torch, paths, max(args.steps, 50))

    yardstick = copy_yardstick(torch, x)
    if args.copy_probe:
        for _ in range(3):
            path.y.copy_(path.x)  # same size as the input tensor
        torch.cuda.synchronize()

    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    q_gbps = q_bytes / (q_med["median_ms"] * 1e-3) / 1e9
    d_gbps = q_bytes / (d_med["median_ms"] * 1e-3) / 1e9
    traffic_table = measured_traffic()
    traffic = traffic_table.get(args.workload, {}).get("quantize_dynamic")

    result = {
        "metric": "quant/dequant GB/s (bytes read+written) and % of MI355X HBM peak, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if w["elem"] == "BF16" else "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {w['desc']}; step = fused dynamic quantize + dequantize",
                   "shape": list(w["shape"]), "block": w["block"], "value": w["value"], "store": "U32",
                   "param": "F32", "algorithmic_bytes_per_step": step_bytes},
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 1),
        "value_note": "algorithmic bytes of the step (each direction: floats + codes + scales once) per second; the "
                      "dequantize of a step reads the codes and scales its quantize has just left in the 256 MB Infinity "
                      "Cache, so fewer bytes than these cross the HBM interface; `roofline` and `roofline_dequantize` time "
                      "each kernel alone on operands from HBM",
        "elements_per_s": round(2 * n / (ms_per_step * 1e-3)),
        # achieved / frac: algorithmic bytes over the MEDIAN launch duration of 50 event-timed regions; the average
        # over one region of K launches (and the regions' mean) stand beside it
        "roofline": {"bound": "hbm", "kernel": "quantize_flat_kernel (fused abs-max+scale+quantize+pack)",
                     "achieved": round(q_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(q_gbps / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "algorithmic_bytes_per_launch": q_bytes, "median_launch_ms": round(q_med["median_ms"], 4),
                     "avg_launch_ms": round(q_ms, 4), "mean_of_regions_ms": round(q_med["mean_ms"], 4),
                     "frac_at_avg": round(q_bytes / (q_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                     "regions": q_med["regions"], "launches_per_region": q_med["launches_per_region"]},
        "roofline_dequantize": {"bound": "hbm", "kernel": "dequantize_flat_kernel", "achieved": round(d_gbps, 1),
                                "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(d_gbps / HBM_PEAK_GBPS, 4),
                                "algorithmic_bytes_per_launch": q_bytes, "median_launch_ms": round(d_med["median_ms"], 4),
                                "avg_launch_ms": round(d_ms, 4),
                                "frac_at_avg": round(q_bytes / (d_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
    }

    for key, name in (("roofline", "quantize"), ("roofline_dequantize", "dequantize")):
        t = in_step[name]
        result[key]["in_step"] = {
            "avg_launch_ms": round(t["avg_launch_ms"], 4), "median_launch_ms": round(t["median_launch_ms"], 4),
            "launches": t["launches"],
            "frac_at_avg": round(q_bytes / (t["avg_launch_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "note": "the launch as the step runs it (quantize, then the dequantize of the same set), one event pair "
                    "per launch; `achieved` and `frac` above are of the kernel alone, back to back on rotated sets"}
    result["copy_yardstick"] = yardstick
    # the headline kernels' bytes: floats on one side, codes + scales on the other
    float_bytes = n * (2 if w["elem"] != "F32" else 4)
    result["memory_yardsticks"] = memory_yardsticks(torch, float_bytes, float_bytes, q_bytes - float_bytes)
    if "additive_ms_quantize" in result["memory_yardsticks"]:
        y = result["memory_yardsticks"]
        result["roofline"]["frac_of_read_plus_write_streams"] = round(y["additive_ms_quantize"] / q_med["median_ms"], 4)
        result["roofline_dequantize"]["frac_of_read_plus_write_streams"] = round(y["additive_ms_dequantize"] / d_med["median_ms"], 4)
    result["first_call_ms"] = {"quantize_dynamic": round(first_ms[0], 2), "dequantize": round(first_ms[1], 2),
                               "library_bytes": os.path.getsize(_ffi.LIB_PATH)}
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, w, path)
        result["cpu_baseline"]["value"] = round(result["cpu_baseline"]["value"], 3)
        result["cpu_baseline"]["elements_per_s"] = round(result["cpu_baseline"]["elements_per_s"])

    if not args.no_sweep:
        table = []
        del path, paths, x
        for name, wk in WORKLOADS.items():
            xi = make_input(torch, wk)
            ps = replicas(torch, wk, xi, min_sets=4)
            b = algorithmic_bytes(wk)
            for p in ps:
                p.compute_scales()
                p.quantize_dynamic()
            row = {"workload": name, "algorithmic_bytes": b, "buffer_sets_rotated": len(ps),
                   # all sets together still fit the 256 MB Infinity Cache: not HBM-bound, reported only
                   "cache_resident": len(ps) * b < (512 << 20)}
            for label in ("quantize_dynamic", "quantize_given_scales", "dequantize"):
                meth = {"quantize_dynamic": "quantize_dynamic", "quantize_given_scales": "quantize_given",
                        "dequantize": "dequantize"}[label]
                fn = lambda i, m=meth: getattr(ps[i % len(ps)], m)()
                med = timed_median(torch, fn)
                med_ms = med["median_ms"]
                row[label] = {"ms": round(med_ms, 4), "mean_ms": round(med["mean_ms"], 4),
                              "GBps": round(b / (med_ms * 1e-3) / 1e9, 1),
                              "frac_hbm_peak": round(b / (med_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                              "traffic": traffic_table.get(name, {}).get(label)}
                if med_ms < 0.016:  # within four host enqueue times: also as a replayed HIP graph
                    row[label]["graph_replay_ms"] = round(graph_region(torch, ps, meth), 4)
            # the two kernels back to back on one buffer set, as in the headline step: the dequantize reads what
            # its quantize has just written
            def both(i, ps=ps):
                ps[i % len(ps)].quantize_dynamic()
                ps[i % len(ps)].dequantize()
            step_ms = sorted(timed_region(torch, both, 32)[0] for _ in range(3))[1]
            row["step_quantize_dynamic_then_dequantize"] = {
                "ms": round(step_ms, 4), "GBps": round(2 * b / (step_ms * 1e-3) / 1e9, 1),
                "sum_of_the_two_alone_ms": round(row["quantize_dynamic"]["ms"] + row["dequantize"]["ms"], 4)}
            del ps, p, xi
            probes = same_traffic_probes(torch, wk)
            if probes is not None:
                row["same_traffic_no_arithmetic"] = probes
                for label, key in (("quantize_dynamic", "quantize_shaped_ms"), ("quantize_given_scales", "quantize_shaped_ms"),
                                   ("dequantize", "dequantize_shaped_ms")):
                    row[label]["frac_of_same_traffic_probe"] = round(probes[key] / row[label]["ms"], 4)
            table.append(row)
        result["per_config"] = table
        # the same fractions where a reader of `roofline` alone finds them: [fused dynamic quantize, quantize with
        # given scales, dequantize] per configuration, median of 50 regions each, and the smallest cell of the three
        # configurations the 70 % target speaks of
        short = {"quantize_dynamic": "dynamic", "quantize_given_scales": "given", "dequantize": "dequantize"}
        result["roofline"]["per_config"] = {
            row["workload"]: {short[k]: row[k]["frac_hbm_peak"] for k in short} for row in table}
        if all("same_traffic_no_arithmetic" in row for row in table):
            # ... and against a launch of the same traffic that computes nothing (probe time / kernel time)
            result["roofline"]["per_config_vs_same_traffic_probe"] = {
                row["workload"]: {short[k]: row[k]["frac_of_same_traffic_probe"] for k in short} for row in table}
        result["roofline"]["min_frac_cfg3_5"] = min(
            row[k]["frac_hbm_peak"] for row in table if row["workload"] in ("cfg3", "cfg4", "cfg5") for k in short)
        result["adjacent_kernels"] = adjacent_kernels(torch) + corner_layouts(torch) + per_tensor_passes(torch) + packed_gemv(torch)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
