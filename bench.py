#!/usr/bin/env python3
"""Benchmark of the ROCm memory component's reduce_multi on one MI355X.

A "step" is one reduce_multi call on the headline workload: FLOAT32 SUM of 8
source vectors of 67,108,864 elements (256 MiB each, stride 256 MiB in one
slab) into a 9th vector -- a radix-8 k-nomial step on 256 MiB buffers.  Inputs
are generated on the device (uniform [-1,1), seeded) and are resident in HBM
before the timed region.  Prints ONE JSON line.

  value            algorithmic GB/s over K steps: K stream-ordered launches
                   (reduce_multi_nb through the dispatcher's C ABI) bracketed
                   by stream synchronisation, bytes = (N+1)*size*4 per step
  roofline         the same bytes / the kernel's average duration -- one HIP
                   event pair on the component's stream around K back-to-back
                   launches -- against 8 TB/s HBM3E; also with the destination
                   rotating through 4 vectors (no reuse of a cached
                   destination) and for 8 x 1 GiB vectors (9+ GiB footprint)
  measured_peak    what this box delivers for a read-only stream with the same
                   access pattern, and for a plain 1:1 copy kernel
  configs          kernel bandwidth of the other benchmark configurations at
                   their full sizes (2-source 1 Mi fp32; the 60-case integer
                   sweep; fp16/fp64 with 16 sources), same timing method
  cpu_baseline     the CPU oracle (port of the reference's host fold, one
                   thread) timed on this box on the same workload
  latency_us       small-message p50/p99 per call in us, FLOAT32 SUM, 2/4/8
                   sources, 4 B .. 32 KiB, 10,000 back-to-back calls each:
                   "sync" = the blocking vtable entry, "event" =
                   reduce_multi_nb + event_query polling (both complete through
                   the kernel's own completion word), "stream" =
                   reduce_multi_nb + hipStreamSynchronize, "graph" =
                   single-node hipGraph launch + hipStreamSynchronize,
                   "issue" = the host's cost of issuing one reduction
  mid_sizes        the scatter-reduce regime (reference allreduce_sra.c:281-284):
                   FLOAT32 SUM, 8 sources x 256 KiB .. 64 MiB per vector, kernel
                   time (region-timed) beside the blocking call a caller sees
"""
import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
N_SRC = 8
SIZE = 67108864
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "reduce_multi_f32_sum_8x256MiB_hbm_traffic.md")
BOX_CPU_SHARE = 16      # host threads a one-GPU job may keep busy on the benchmark boxes


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--size", type=int, default=SIZE, help="elements per vector (default: the headline 67,108,864)")
    ap.add_argument("--nsrc", type=int, default=N_SRC)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-latency", action="store_true", help="skip the small-message sweep")
    ap.add_argument("--no-configs", action="store_true", help="skip the other benchmark configurations")
    ap.add_argument("--latency-iters", type=int, default=10000)
    ap.add_argument("--latency-quick", action="store_true", help="3 of the 14 message sizes only")
    ap.add_argument("--profile-mode", nargs="?", const="headline", default=None,
                    choices=("headline", "footprint", "config3_int8", "config4_f16", "config4_f64", "small"),
                    help="for rocprofv3: only K launches of the named workload (headline: followed by K launches of a "
                         "1 GiB + 1 GiB copy kernel, the known-traffic calibration), nothing else")
    ap.add_argument("--matrix", action="store_true",
                    help="kernel GB/s of every benchmark configuration, row by row (all dtype/op pairs of the integer "
                         "sweep and the 16-source cases included); table to <out-dir>/matrix.json, nothing else")
    ap.add_argument("--replay", action="store_true",
                    help="time whole allreduce collectives of the replayed UCX call sites (8 loopback ranks on the one "
                         "GPU): blocking reductions as in the reference vs stream-ordered ones, scratch cached vs not")
    ap.add_argument("--latency-child", action="store_true",
                    help="a handful of small-message rows as JSON and nothing else (the default run starts this in a "
                         "child process whose runtime keeps its queue rings in device memory)")
    ap.add_argument("--out-dir", default=os.path.join(ROOT, "bench_out"), help="where --matrix / --replay write")
    return ap.parse_args()


def region_gbps(mc, buf, nsrc, size, es, dt, op, iters, rbuf=None, rot=0):
    """Algorithmic GB/s and average launch duration (us): one event pair around `iters` back-to-back launches."""
    from xccl_amd.types import Status
    stride = size * es
    nb = (nsrc + 1) * stride
    rbuf = buf + nsrc * stride if rbuf is None else rbuf
    if rot:
        st, ms = mc.bench_region_time_rot(buf, buf + stride, rbuf, rot, stride, nsrc - 1, size, stride, dt, op, iters)
    else:
        st, ms = mc.bench_region_time(buf, buf + stride, rbuf, nsrc - 1, size, stride, dt, op, iters)
    assert st == Status.OK, st
    return nb * iters / ms / 1e6, ms / iters * 1e3


def entry(gbps, us, nb, **kw):
    d = {"achieved": round(gbps, 1), "unit": "GB/s", "peak": HBM_PEAK_GBPS, "frac": round(gbps / HBM_PEAK_GBPS, 4),
         "bound": "hbm", "kernel_us_avg": round(us, 2), "bytes_per_launch": nb}
    d.update(kw)
    return d


def cpu_baseline(size, nsrc):
    """The oracle's fold on the same workload, host memory: one thread (what one reference rank does), and
    the same function on disjoint chunks by as many threads as the box lets a one-GPU job keep busy."""
    from oracle import pyoracle as o
    from xccl_amd.types import Dt, Op
    host_cpus = os.cpu_count() or 1
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = host_cpus
    threads = max(1, min(BOX_CPU_SHARE, usable))
    slab = o.slab(nsrc, size, Dt.FLOAT32, 2, threads=threads)
    out = np.empty(size, dtype=np.float32)
    nbytes = (nsrc + 1) * size * 4
    stride = size * 4

    def run(th):
        t0 = time.perf_counter()
        o.reduce_multi(slab, slab, out, nsrc - 1, size, stride, Dt.FLOAT32, Op.SUM, off2=stride, threads=th)
        return time.perf_counter() - t0

    run(1)
    t1 = []
    while sum(t1) < 10.0 and len(t1) < 200:
        t1.append(run(1))
    run(threads)
    tm = []
    while sum(tm) < 4.0 and len(tm) < 20:
        tm.append(run(threads))
    med1, medm = float(np.median(t1)), float(np.median(tm))
    # the reference's own CPU-runnable case: xccl_dt_reduce on two 4 MiB fp32 vectors, one thread
    n1 = 1 << 20
    a1, b1, o1 = o.fill(n1, Dt.FLOAT32, 0, 0), o.fill(n1, Dt.FLOAT32, 0, 1), np.empty(n1, dtype=np.float32)
    tc = []
    for _ in range(200):
        t0 = time.perf_counter()
        o.dt_reduce(a1, b1, o1, n1, Dt.FLOAT32, Op.SUM)
        tc.append(time.perf_counter() - t0)
    medc = float(np.median(tc[20:]))
    return {
        "value": round(nbytes / med1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": "%d calls of the full workload (%d x %d fp32, %d B/call, %.1f s of CPU work), median %.1f ms/call; "
                  "host traffic is 3*(N-1)*size*4 B/call" % (len(t1), nsrc, size, nbytes, sum(t1), med1 * 1e3),
        "host_cpu_count": host_cpus, "usable_cpus": usable,
        "all_cores": {"value": round(nbytes / medm / 1e9, 3), "cores": threads, "ms_per_call": round(medm * 1e3, 2),
                      "note": "one thread per core of the %d-core share a one-GPU job has on the box "
                              "(os.cpu_count() = %d)" % (BOX_CPU_SHARE, host_cpus)},
        "two_source_1Mi_fp32": {"value": round(3 * n1 * 4 / medc / 1e9, 3), "unit": "GB/s", "cores": 1,
                                "us_per_call": round(medc * 1e6, 1)},
    }, slab, out


def latency_sweep(mc, hip, iters, quick):
    """Config 5: FLOAT32 SUM, 2/4/8 sources, 4 B .. 32 KiB per vector, `iters` back-to-back calls per cell."""
    from xccl_amd.types import Dt, Op, Status
    sizes_b = [4, 1024, 32768] if quick else [4 << k for k in range(14)]
    res = {"iterations_per_cell": iters, "bytes_per_vector": sizes_b,
           "modes": {"sync": "blocking vtable entry (launches on the component's own dispatch queue)",
                     "event": "reduce_multi_nb + event_query until done (own dispatch queue)",
                     "issue": "reduce_multi_nb with an event: host time of the call alone",
                     "sync_on_hip_stream": "blocking vtable entry with the own queue switched off: hipLaunchKernel on "
                                           "the component's stream, completion word",
                     "stream": "reduce_multi_nb without an event + hipStreamSynchronize",
                     "graph": "cached one-node hipGraph launch + hipStreamSynchronize"}}
    maxb = 32768
    buf = hip.DeviceBuffer(10 * maxb)
    for j in range(9):
        mc.datagen_fill(buf.ptr + j * maxb, maxb // 4, Dt.FLOAT32, 5, j)
    hip.device_synchronize()
    for nsrc in (2, 4, 8):
        for b in sizes_b:
            cnt = b // 4
            row = {}
            for mode in ("sync", "event", "stream", "graph", "issue"):
                n = iters if mode != "graph" else max(1000, iters // 4)     # a graph launch takes ~4x as long
                st, ns = mc.bench_latency(mode, buf.ptr, buf.ptr + maxb, buf.ptr + 9 * maxb, nsrc - 1, cnt, maxb,
                                          Dt.FLOAT32, Op.SUM, n)
                assert st == Status.OK, (mode, st)
                ns = ns[n // 10:]
                row[mode] = {"p50": round(float(np.percentile(ns, 50)) / 1e3, 2),
                             "p99": round(float(np.percentile(ns, 99)) / 1e3, 2)}
            # the blocking entry once more with the component's own dispatch queue switched off: the same launch
            # through hipLaunchKernel on the component's stream
            mc.component_lib().xccl_rocm_set_direct_queue(0)
            st, ns = mc.bench_latency("sync", buf.ptr, buf.ptr + maxb, buf.ptr + 9 * maxb, nsrc - 1, cnt, maxb,
                                      Dt.FLOAT32, Op.SUM, iters)
            mc.component_lib().xccl_rocm_set_direct_queue(1)
            assert st == Status.OK, st
            ns = ns[iters // 10:]
            row["sync_on_hip_stream"] = {"p50": round(float(np.percentile(ns, 50)) / 1e3, 2),
                                         "p99": round(float(np.percentile(ns, 99)) / 1e3, 2)}
            res["n%d_%dB" % (nsrc, b)] = row
    # where the time of a one-node graph launch goes (4 sources x 1 KiB, completion word carried by the graph)
    st, parts = mc.bench_graph_parts(buf.ptr, buf.ptr + maxb, buf.ptr + 9 * maxb, 3, 256, maxb, Dt.FLOAT32, Op.SUM, 3000)
    assert st == Status.OK, st
    p = np.percentile(parts[300:].astype(np.float64), 50, axis=0) / 1e3
    res["graph_launch_steps_n4_1024B_p50"] = {
        "planning": round(float(p[0]), 2), "lock_and_slot_search": round(float(p[1]), 2),
        "patch_node_params": round(float(p[2]), 2), "hipGraphLaunch": round(float(p[3]), 2),
        "launch_returned_to_completion_word_seen": round(float(p[4]), 2), "whole_call": round(float(p[5]), 2)}
    return res, buf


def mid_sizes(mc, hip):
    """FLOAT32 SUM, 8 sources x 256 KiB .. 64 MiB per vector (powers of 4): average kernel duration (one event
    pair around 200 back-to-back launches on the component's stream) and what a caller of the blocking entry
    sees per call (host clock, p50 of 200 calls), both also as algorithmic GB/s."""
    from xccl_amd.types import Dt, MemType, Op, Status
    rows = {}
    nsrc = 8
    for vb in (256 << 10, 1 << 20, 4 << 20, 16 << 20, 64 << 20):
        size = vb // 4
        nb = (nsrc + 1) * vb
        st, slab = mc.xccl_mem_component_alloc(nb, MemType.ROCM)
        assert st == Status.OK, st
        for j in range(nsrc):
            assert mc.datagen_fill(slab + j * vb, size, Dt.FLOAT32, 4, j) == Status.OK
        hip.device_synchronize()
        region_gbps(mc, slab, nsrc, size, 4, Dt.FLOAT32, Op.SUM, 20)
        g, us = region_gbps(mc, slab, nsrc, size, 4, Dt.FLOAT32, Op.SUM, 200)
        route = mc.reduce_multi_route(slab, slab + vb, slab + nsrc * vb, nsrc - 1, size, vb, Dt.FLOAT32, Op.SUM, True)
        if route["route"] == "stream":      # too large for the own queue: what the HIP stream path does with it
            route = mc.reduce_multi_route(slab, slab + vb, slab + nsrc * vb, nsrc - 1, size, vb, Dt.FLOAT32, Op.SUM, False)
            where = "hip stream"
        else:
            where = "own queue"
        st, ns = mc.bench_latency("sync", slab, slab + vb, slab + nsrc * vb, nsrc - 1, size, vb, Dt.FLOAT32, Op.SUM, 220)
        assert st == Status.OK, st
        call_us = float(np.percentile(ns[20:], 50)) / 1e3
        rows["n8_%dKiB" % (vb >> 10)] = {
            "bytes_per_call": nb, "kernel_us": round(us, 2), "kernel_GBps": round(g, 1),
            "blocking_call_us": round(call_us, 2), "blocking_call_p99_us": round(float(np.percentile(ns[20:], 99)) / 1e3, 2),
            "blocking_call_GBps": round(nb / call_us / 1e3, 1), "call_minus_kernel_us": round(call_us - us, 2),
            "launched_on": where, "completion": route["route"], "grid": route["grid"]}
        mc.xccl_mem_component_free(slab, MemType.ROCM)
    return rows


def latency_child(mc, hip, iters):
    """A few rows of the small-message sweep: blocking entry, 2/4/8 sources, and 1/2/4 calling threads."""
    from xccl_amd.types import Dt, Op, Status
    res = {}
    maxb = 32768
    buf = hip.DeviceBuffer(10 * maxb)
    for j in range(9):
        mc.datagen_fill(buf.ptr + j * maxb, maxb // 4, Dt.FLOAT32, 5, j)
    hip.device_synchronize()
    for nsrc, b in ((2, 4), (4, 1024), (8, 1024), (8, 32768)):
        st, ns = mc.bench_latency("sync", buf.ptr, buf.ptr + maxb, buf.ptr + 9 * maxb, nsrc - 1, b // 4, maxb, Dt.FLOAT32,
                                  Op.SUM, iters)
        assert st == Status.OK, st
        ns = ns[iters // 10:]
        res["n%d_%dB" % (nsrc, b)] = {"p50": round(float(np.percentile(ns, 50)) / 1e3, 2),
                                      "p99": round(float(np.percentile(ns, 99)) / 1e3, 2)}
    tb = hip.DeviceBuffer(8 * 8192)
    for th in (1, 2, 4):
        st, ns = mc.bench_latency_mt(th, 8192, tb.ptr, tb.ptr + 1024, tb.ptr + 4096, 3, 256, 1024, Dt.FLOAT32, Op.SUM,
                                     iters)
        assert st == Status.OK
        ns = ns[:, iters // 10:]
        res["threads%d_n4_1024B" % th] = {"p50": round(float(np.percentile(ns, 50)) / 1e3, 2),
                                          "p99": round(float(np.percentile(ns, 99)) / 1e3, 2)}
    tb.close()
    buf.close()
    return res


def latency_with_runtime_queues_in_device_memory(iters):
    """The same rows from a child process started with HSA_ALLOCATE_QUEUE_DEV_MEM=1: the HSA runtime then keeps
    the packet rings of every queue it creates, the component's own included, in device memory, and the packet
    processor no longer fetches a packet over PCIe.  A process-wide setting of the runtime, read when it
    initialises: a deployment's choice, not something a plugin can switch on for its host."""
    import subprocess
    env = dict(os.environ, HSA_ALLOCATE_QUEUE_DEV_MEM="1")
    out = subprocess.run([sys.executable, os.path.abspath(__file__), "--latency-child", "--latency-iters", str(iters)],
                         env=env, capture_output=True, text=True, timeout=300)
    if out.returncode != 0:
        return {"error": (out.stderr or out.stdout)[-300:]}
    res = json.loads(out.stdout.strip().splitlines()[-1])
    res["setting"] = "HSA_ALLOCATE_QUEUE_DEV_MEM=1 in the environment of a child process; blocking entry, p50 / p99 in us"
    return res


def latency_extras(mc, hip, buf, iters):
    from xccl_amd.types import Dt, Op, Status
    res = {}
    # blocking calls from several host threads at once (XCCL_THREAD_MODE_MULTIPLE, reference test/test_mt.c):
    # 4 sources x 1 KiB, every thread on operands of its own
    tb = hip.DeviceBuffer(8 * 8192)
    for th in (1, 2, 4):
        st, ns = mc.bench_latency_mt(th, 8192, tb.ptr, tb.ptr + 1024, tb.ptr + 4096, 3, 256, 1024, Dt.FLOAT32, Op.SUM,
                                     iters)
        assert st == Status.OK
        ns = ns[:, iters // 10:]
        res["threads%d_n4_1024B" % th] = {"p50": round(float(np.percentile(ns, 50)) / 1e3, 2),
                                          "p99": round(float(np.percentile(ns, 99)) / 1e3, 2)}
    # a small blocking call with a system-scope acquire fence on the own queue's packets instead of the agent-scope one
    lib = mc.component_lib()
    for scope, flag in (("agent", 0), ("system", 1)):
        lib.xccl_rocm_set_direct_options(flag, -1, -1, -1, -1)
        for nsrc, nbv in ((4, 1024), (8, 32768)):
            st, ns = mc.bench_latency("sync", buf.ptr, buf.ptr + 32768, buf.ptr + 9 * 32768, nsrc - 1, nbv // 4, 32768,
                                      Dt.FLOAT32, Op.SUM, iters)
            assert st == Status.OK
            ns = ns[iters // 10:]
            res["acquire_%s_n%d_%dB" % (scope, nsrc, nbv)] = {"p50": round(float(np.percentile(ns, 50)) / 1e3, 2),
                                                              "p99": round(float(np.percentile(ns, 99)) / 1e3, 2)}
    lib.xccl_rocm_set_direct_options(0, -1, -1, -1, -1)
    tb.close()
    # memcpy_async + event_record + event_query: one message of the loopback transport / one mpod alltoall step
    ms = mc.Stream(hip.stream_create())
    cb = hip.DeviceBuffer(2 << 20)
    for nb in (1024, 65536, 1 << 20):
        st, ns = mc.bench_memcpy(ms, cb.ptr, cb.ptr + (1 << 20), nb, 1000)
        assert st == Status.OK
        res["memcpy_event_%dB" % nb] = {"p50": round(float(np.percentile(ns[100:], 50)) / 1e3, 2),
                                        "p99": round(float(np.percentile(ns[100:], 99)) / 1e3, 2)}
    hip.stream_synchronize(ms.hip_stream)
    hip.stream_destroy(ms.hip_stream)
    cb.close()
    # the memory-type probe libxccl issues at least twice per collective (mem_component.c:150-174)
    host = np.zeros(16, dtype=np.uint8)
    for name, ptr in (("device", buf.ptr), ("unregistered_host", host.ctypes.data)):
        st, ns, mt = mc.bench_mem_type(ptr, 2000)
        assert st == Status.OK
        res["mem_type_probe_" + name] = {"p50": round(float(np.percentile(ns[200:], 50)) / 1e3, 3),
                                         "p99": round(float(np.percentile(ns[200:], 99)) / 1e3, 3),
                                         "answer": mt.name if mt is not None else "not recognised"}
    # scratch per collective: mem_alloc + mem_free through the vtable, freed blocks cached (default) or not
    for label, limit in (("cached", 8 << 30), ("runtime", 0)):
        mc.mem_pool_set_limit(limit)
        for nb in (64 << 10, 1 << 20, 64 << 20, 7 * 256 << 20):    # last: scratch of the headline radix-8 step
            st, ns = mc.bench_alloc_free(nb, 300 if nb <= (64 << 20) else 60)
            assert st == Status.OK
            res["alloc_free_%s_%dKiB" % (label, nb >> 10)] = {
                "p50": round(float(np.percentile(ns[10:], 50)) / 1e3, 3),
                "p99": round(float(np.percentile(ns[10:], 99)) / 1e3, 3)}
    mc.mem_pool_set_limit(8 << 30)
    return res


def config_cases():
    from xccl_amd.types import Dt, Op, INT_OPS
    cases = [("config1", Dt.FLOAT32, Op.SUM, 2, 1048576)]
    for dt in (Dt.INT8, Dt.INT16, Dt.INT32, Dt.INT64, Dt.UINT32, Dt.UINT64):
        cases += [("config3", dt, op, 4, 16777216) for op in INT_OPS]
    for dt in (Dt.FLOAT16, Dt.FLOAT64):
        cases += [("config4", dt, op, 16, 33554432) for op in (Op.SUM, Op.MAX, Op.MIN)]
    return cases


class Slab:
    """Device slab of nsrc + extra vectors, refilled only when the (dtype, shape, zero-rich) key changes."""

    def __init__(self, mc, hip):
        self.mc, self.hip, self.key, self.buf = mc, hip, None, None

    def get(self, dt, nsrc, size, sparse, extra=1):
        from xccl_amd.types import MemType, Status, dt_size
        key = (dt, nsrc, size, sparse, extra)
        if key != self.key:
            self.close()
            stride = size * dt_size(dt)
            st, self.buf = self.mc.xccl_mem_component_alloc((nsrc + extra) * stride, MemType.ROCM)
            assert st == Status.OK, st
            for j in range(nsrc):
                assert self.mc.datagen_fill(self.buf + j * stride, size, dt, 3, j, sparse) == Status.OK
            self.hip.device_synchronize()
            self.key = key
        return self.buf

    def close(self):
        from xccl_amd.types import MemType
        if self.buf is not None:
            self.mc.xccl_mem_component_free(self.buf, MemType.ROCM)
        self.buf, self.key = None, None


def run_configs(mc, hip):
    """Kernel bandwidth of configurations 1, 3 and 4 at their full sizes.  Short kernels are timed like the
    headline: one event pair around many back-to-back launches."""
    from xccl_amd.types import Op, dt_size
    slab = Slab(mc, hip)
    rows = []
    for name, dt, op, nsrc, size in config_cases():
        es = dt_size(dt)
        nb = (nsrc + 1) * size * es
        buf = slab.get(dt, nsrc, size, op in (Op.LAND, Op.LOR, Op.LXOR))
        iters = max(20, min(400, int(8e9 // nb)))
        region_gbps(mc, buf, nsrc, size, es, dt, op, 3)
        g, us = region_gbps(mc, buf, nsrc, size, es, dt, op, iters)
        rows.append((name, dt, op, nsrc, size, nb, g, us, iters))
    slab.close()
    out = {}
    r = rows[0]
    out["config1"] = entry(r[6], r[7], r[5], workload="FLOAT32 SUM, 2 sources x 1,048,576 elements (device)",
                           launches_timed=r[8])
    c3 = {}
    for dt in sorted({r[1] for r in rows if r[0] == "config3"}, key=int):
        rs = [r for r in rows if r[0] == "config3" and r[1] == dt]
        fr = sorted(x[6] for x in rs)
        worst = min(rs, key=lambda x: x[6])
        c3[dt.name] = {"bound": "hbm", "unit": "GB/s", "peak": HBM_PEAK_GBPS, "bytes_per_launch": rs[0][5],
                       "min": round(fr[0], 1), "median": round(float(np.median(fr)), 1), "max": round(fr[-1], 1),
                       "frac_min": round(fr[0] / HBM_PEAK_GBPS, 4),
                       "frac_median": round(float(np.median(fr)) / HBM_PEAK_GBPS, 4),
                       "slowest_op": worst[2].name, "kernel_us_avg_slowest": round(worst[7], 2),
                       "per_op": {x[2].name: round(x[6], 1) for x in rs}, "launches_timed": rs[0][8]}
    out["config3"] = {"workload": "4 sources x 16,777,216 elements, 10 operators per dtype; vectors of 16-128 MiB: "
                                  "the 1- and 2-byte cases fit the 256 MB memory-side cache", "per_dtype": c3}
    c4 = {}
    for r in rows:
        if r[0] == "config4":
            c4["%s_%s" % (r[1].name, r[2].name)] = entry(r[6], r[7], r[5], launches_timed=r[8])
    out["config4"] = {"workload": "16 sources x 33,554,432 elements (radix-16 step)", "cases": c4}
    return out


def matrix(mc, hip, out_dir):
    """Region-timed kernel bandwidth of each benchmark configuration at its full size, plus extras."""
    from xccl_amd.types import Dt, Op, Status, dt_size
    cases = config_cases()
    cases.insert(1, ("config2", Dt.FLOAT32, Op.SUM, 8, 67108864))
    cases += [("extra", Dt.FLOAT32, Op.SUM, n, 67108864) for n in (2, 3, 4, 5, 16)]
    cases += [("extra", Dt.UINT8, op, 4, 67108864) for op in (Op.SUM, Op.MAX)]
    cases += [("extra", Dt.FLOAT16, Op.PROD, 8, 67108864), ("extra", Dt.FLOAT32, Op.MAX, 8, 67108864)]
    cases += [("inplace", Dt.FLOAT32, Op.MAX, n, 67108864) for n in (4, 8)]
    # message-size sweep: where the call leaves the launch-bound regime and reaches the bandwidth plateau
    cases += [("sweep", Dt.FLOAT32, Op.SUM, n, 1 << k) for n in (2, 4, 8) for k in range(14, 27, 2)]
    rows = []
    slab = Slab(mc, hip)
    for name, dt, op, nsrc, size in cases:
        es = dt_size(dt)
        stride = size * es
        nb = (nsrc + 1) * stride
        buf = slab.get(dt, nsrc, size, op in (Op.LAND, Op.LOR, Op.LXOR), extra=4)
        # "inplace": rbuf == sbuf1, the form every k-nomial round after the first has (allreduce_knomial.c:118-121)
        rbuf = buf if name == "inplace" else buf + nsrc * stride
        iters = max(20, min(400, int(8e9 // nb)))
        region_gbps(mc, buf, nsrc, size, es, dt, op, 3, rbuf=rbuf)
        g, us = region_gbps(mc, buf, nsrc, size, es, dt, op, iters, rbuf=rbuf)
        row = {"config": name, "dtype": dt.name, "op": op.name, "nsrc": nsrc, "size": size, "bytes": nb,
               "kernel_us": round(us, 2), "GBps": round(g, 1), "frac_of_peak": round(g / HBM_PEAK_GBPS, 3)}
        if name not in ("inplace", "sweep"):
            gr, _ = region_gbps(mc, buf, nsrc, size, es, dt, op, iters, rot=4)
            row["GBps_rotating_dst"] = round(gr, 1)
        if name == "sweep":     # what a caller of the blocking entry sees per call, host clock
            st, ns = mc.bench_latency("sync", buf, buf + stride, buf + nsrc * stride, nsrc - 1, size, stride, dt, op,
                                      200)
            assert st == Status.OK
            row["blocking_call_us"] = round(float(np.percentile(ns[20:], 50)) / 1e3, 2)
            row["blocking_call_GBps"] = round(nb / row["blocking_call_us"] / 1e3, 1)
        rows.append(row)
        print("%-8s %-8s %-5s N=%-2d size=%-9d %9.2f us %8.1f GB/s %s" % (
            name, dt.name, op.name, nsrc, size, us, g,
            "blocking call %.2f us" % row["blocking_call_us"] if name == "sweep" else
            "rotating %.1f" % row.get("GBps_rotating_dst", 0)), file=sys.stderr, flush=True)
    slab.close()
    os.makedirs(out_dir, exist_ok=True)
    json.dump(rows, open(os.path.join(out_dir, "matrix.json"), "w"), indent=1)
    print(json.dumps({"matrix_rows": len(rows),
                      "min_GBps": min(r["GBps"] for r in rows if r["config"] not in ("config1", "sweep", "inplace")),
                      "file": os.path.join(out_dir, "matrix.json")}))
    return 0


def replay_bench(mc, hip, out_dir):
    """Whole-collective times of the replayed call sites.  The loopback transport moves bytes with device
    copies, so the figures show what the reduction path and the scratch allocation contribute to a
    collective, not what a network would."""
    from xccl_amd.types import Dt, Op, Status
    P = 8
    rows = []
    for count in (256, 16384, 1 << 20, 1 << 24):
        nb = count * 4
        src = [hip.DeviceBuffer(nb) for _ in range(P)]
        dst = [hip.DeviceBuffer(nb) for _ in range(P)]
        for r in range(P):
            assert mc.datagen_fill(src[r].ptr, count, Dt.FLOAT32, 9, r) == Status.OK
        hip.device_synchronize()
        for alg, radix in (("allreduce_knomial", 4), ("allreduce_knomial", 8), ("allreduce_sra", 4)):
            for mode, pool in (("blocking", 0), ("blocking", 8 << 30), ("stream_ordered", 8 << 30)):
                mc.mem_pool_set_limit(pool)
                ts = []
                for it in range(35):
                    t0 = time.perf_counter()
                    st, stats = mc.replay_run(alg, [b.ptr for b in src], [b.ptr for b in dst], count, Dt.FLOAT32,
                                              Op.SUM, radix=radix, stream_ordered=(mode == "stream_ordered"))
                    ts.append(time.perf_counter() - t0)
                    assert st == Status.OK, (alg, radix, mode, st)
                ts = np.array(ts[5:]) * 1e6
                rows.append({"alg": alg, "ranks": P, "radix": radix, "bytes_per_rank": nb, "reductions": mode,
                             "scratch": "cached" if pool else "runtime alloc/free",
                             "p50_us": round(float(np.percentile(ts, 50)), 1),
                             "p90_us": round(float(np.percentile(ts, 90)), 1),
                             "reduce_calls": stats["reduce_calls"] + stats["reduce_multi_calls"],
                             "inflight_returns": stats["reduce_inflight_returns"]})
                print("%-18s radix %d %9d B  %-14s %-18s p50 %9.1f us" % (alg, radix, nb, mode, rows[-1]["scratch"],
                                                                        rows[-1]["p50_us"]), file=sys.stderr, flush=True)
        for b in src + dst:
            b.close()
    mc.mem_pool_set_limit(8 << 30)
    os.makedirs(out_dir, exist_ok=True)
    json.dump(rows, open(os.path.join(out_dir, "replay.json"), "w"), indent=1)
    print(json.dumps({"replay_rows": len(rows), "file": os.path.join(out_dir, "replay.json")}))
    return 0


def profile_mode(a, mc, hip):
    """Only the launches rocprofv3 is meant to see."""
    from xccl_amd.types import Dt, MemType, Op, Status, dt_size
    work = {"headline": (Dt.FLOAT32, Op.SUM, 8, SIZE), "footprint": (Dt.FLOAT32, Op.SUM, 8, 1 << 28),
            "config3_int8": (Dt.INT8, Op.PROD, 4, 16777216),
            "config4_f16": (Dt.FLOAT16, Op.SUM, 16, 33554432), "config4_f64": (Dt.FLOAT64, Op.SUM, 16, 33554432),
            "small": (Dt.FLOAT32, Op.SUM, 4, 256)}[a.profile_mode]
    dt, op, nsrc, size = work
    es = dt_size(dt)
    stride = size * es
    slab = Slab(mc, hip)
    # "footprint": 8 x 1 GiB sources, the destination rotating through 4 more vectors (12 GiB touched)
    rot = 4 if a.profile_mode == "footprint" else 1
    buf = slab.get(dt, nsrc, size, False, extra=rot)
    stream = mc.component_stream()
    n = a.warmup + a.steps
    for i in range(n):
        st_, _ = mc.xccl_mem_component_reduce_multi_nb(buf, buf + stride, buf + (nsrc + i % rot) * stride, nsrc - 1, size,
                                                       stride, dt, op, MemType.ROCM, None, want_event=False)
        assert st_ == Status.OK
    hip.stream_synchronize(stream)
    info = {"profile_mode": a.profile_mode, "reduce_launches": n, "dtype": dt.name, "op": op.name, "nsrc": nsrc,
            "size": size, "reduce_algorithmic_bytes": (nsrc + 1) * stride}
    info.update(plan_of(mc, buf, nsrc, size, stride, dt, op))
    if a.profile_mode == "footprint":
        for _ in range(n):     # the reduction's reads without its store, same residency bound
            assert mc.bench_read(buf, stride, nsrc, stride, 10240, stream) == Status.OK
        hip.stream_synchronize(stream)
        info.update({"read_only_launches": n, "read_only_bytes": nsrc * stride, "destinations": rot})
    if a.profile_mode == "headline":
        gib = 1 << 30
        for _ in range(n):     # sources 0-3 -> sources 4-7: reads 1 GiB, writes 1 GiB
            assert mc.bench_copy(buf + 4 * stride, buf, gib, stream) == Status.OK
        hip.stream_synchronize(stream)
        for _ in range(n):     # the reduction's reads without its store
            assert mc.bench_read(buf, stride, nsrc, stride, 10240, stream) == Status.OK
        hip.stream_synchronize(stream)
        info.update({"copy_launches": n, "copy_bytes_read": gib, "copy_bytes_written": gib, "read_only_launches": n,
                     "read_only_bytes": nsrc * stride})
    slab.close()
    print(json.dumps(info))
    return 0


def plan_of(mc, buf, nsrc, size, stride, dt, op):
    return mc.reduce_multi_plan(buf, buf + stride, buf + nsrc * stride, nsrc - 1, size, stride, dt, op)


def traffic_for(plan):
    """HBM bytes per launch measured with rocprofv3 counters for exactly this kernel and grid, else None: the
    committed summary names the kernel and grid it was measured on."""
    if not os.path.isfile(TRAFFIC_FILE):
        return None
    text = open(TRAFFIC_FILE).read()
    got = {}
    for key in ("kernel", "grid", "bytes_per_launch"):
        m = re.search(r"^%s:\s*(\S+)" % key, text, flags=re.M)
        if not m:
            return None
        got[key] = m.group(1)
    if got["kernel"] != plan["kernel"] or int(got["grid"]) != plan["grid"]:
        return None
    return int(float(got["bytes_per_launch"]))


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the reduction path is local arithmetic between p2p rounds; "
              "no inter-GPU work exists to scale) -- use --gpus 1", file=sys.stderr)
        return 2

    from xccl_amd import build, hip, mc
    from xccl_amd.types import Dt, MemType, Op, Status

    if not build.built():          # load what is built; compile only if nothing is
        build.build(force=False)
    if hip.device_count() < 1:
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    hip.set_device(0)
    assert mc.xccl_mem_component_init() == Status.OK
    assert bool(mc.dispatch_lib().xccl_mem_component_get(int(MemType.ROCM))), "ROCm component not loaded"

    if a.latency_child:
        print(json.dumps(latency_child(mc, hip, min(a.latency_iters, 4000))))
        return 0
    if a.matrix:
        return matrix(mc, hip, a.out_dir)
    if a.replay:
        return replay_bench(mc, hip, a.out_dir)
    if a.profile_mode:
        return profile_mode(a, mc, hip)

    size, nsrc = a.size, a.nsrc
    stride = size * 4
    nbytes = (nsrc + 1) * size * 4
    st, slab = mc.xccl_mem_component_alloc((nsrc + 4) * stride, MemType.ROCM)   # 8 sources + 4 destinations
    assert st == Status.OK
    dst = slab + nsrc * stride
    for j in range(nsrc):
        assert mc.datagen_fill(slab + j * stride, size, Dt.FLOAT32, 2, j) == Status.OK
    hip.device_synchronize()
    stream = mc.component_stream()

    def step():
        st_, _ = mc.xccl_mem_component_reduce_multi_nb(slab, slab + stride, dst, nsrc - 1, size, stride, Dt.FLOAT32,
                                                       Op.SUM, MemType.ROCM, None, want_event=False)
        assert st_ == Status.OK

    for _ in range(a.warmup):
        step()
    hip.stream_synchronize(stream)
    hip.device_synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    hip.stream_synchronize(stream)
    hip.device_synchronize()
    dt_total = time.perf_counter() - t0
    ms_per_step = dt_total / a.steps * 1e3
    gbps = nbytes / (dt_total / a.steps) / 1e9

    # the blocking vtable entry (launch + wait inside), for comparison
    t0 = time.perf_counter()
    for _ in range(a.steps):
        assert mc.xccl_mem_component_reduce_multi(slab, slab + stride, dst, nsrc - 1, size, stride, Dt.FLOAT32, Op.SUM,
                                                  MemType.ROCM) == Status.OK
    sync_ms = (time.perf_counter() - t0) / a.steps * 1e3

    # average launch duration: one event pair on the kernel's own stream around K back-to-back launches
    k = max(a.steps, 10)
    achieved, k_us = region_gbps(mc, slab, nsrc, size, 4, Dt.FLOAT32, Op.SUM, k)
    # ... with the destination cycling through 4 vectors (1 GiB), so that the 256 MiB destination cannot
    # stay resident in the 256 MB memory-side cache between launches (footprint 3.25 GiB)
    region_gbps(mc, slab, nsrc, size, 4, Dt.FLOAT32, Op.SUM, 4, rot=4)
    rot, rot_us = region_gbps(mc, slab, nsrc, size, 4, Dt.FLOAT32, Op.SUM, k, rot=4)
    # ... and with an event pair around each launch, for comparison (the pair costs ~5 us on this part)
    st, kms = mc.bench_kernel_times(slab, slab + stride, dst, nsrc - 1, size, stride, Dt.FLOAT32, Op.SUM, k)
    assert st == Status.OK
    plan = plan_of(mc, slab, nsrc, size, stride, Dt.FLOAT32, Op.SUM)

    # What the box delivers: a read-only stream with the reduction's access pattern, and a plain copy kernel.
    peak = {}
    if nsrc >= 8 and stride * 4 >= (1 << 30):
        e0, e1 = hip.event_create(), hip.event_create()
        for lds, label in ((10240, "read_only_GBps"), (0, "read_only_no_residency_cap_GBps")):
            for _ in range(3):
                assert mc.bench_read(slab, stride, nsrc, stride, lds, stream) == Status.OK
            hip.event_record(e0, stream)
            for _ in range(20):
                assert mc.bench_read(slab, stride, nsrc, stride, lds, stream) == Status.OK
            hip.event_record(e1, stream)
            hip.event_synchronize(e1)
            peak[label] = round(nsrc * stride * 20 / hip.event_elapsed_ms(e0, e1) / 1e6, 1)
        gib = 1 << 30
        for _ in range(3):
            assert mc.bench_copy(slab + 8 * stride, slab, gib, stream) == Status.OK     # sources 0-3 -> destinations
        hip.event_record(e0, stream)
        for _ in range(20):
            assert mc.bench_copy(slab + 8 * stride, slab, gib, stream) == Status.OK
        hip.event_record(e1, stream)
        hip.event_synchronize(e1)
        peak["copy_kernel_GBps"] = round(2 * gib * 20 / hip.event_elapsed_ms(e0, e1) / 1e6, 1)
        peak["note"] = "read_only: the reduction's walk over 8 x 256 MiB without the store; copy: 1 GiB -> 1 GiB, " \
                       "bytes read + written"
        hip.event_destroy(e0)
        hip.event_destroy(e1)
        assert mc.xccl_mem_component_reduce_multi(slab, slab + stride, dst, nsrc - 1, size, stride, Dt.FLOAT32, Op.SUM,
                                                  MemType.ROCM) == Status.OK

    out = {
        "metric": "reduce_multi GB/s (fp32 sum, %d srcs x %d MiB)" % (nsrc, stride >> 20),
        "value": round(gbps, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "reduce_multi FLOAT32 SUM, %d source vectors x %d elements at stride %d B in one slab "
                               "(radix-8 k-nomial step); stream-ordered launches" % (nsrc, size, stride),
                   "bytes_per_step": nbytes, "device": "gfx950 (%s)" % hip.device_name(0),
                   "kernel": plan["kernel"], "grid": plan["grid"], "block": plan["block"]},
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "sync_entry": {"ms_per_step": round(sync_ms, 4), "GBps": round(nbytes / sync_ms / 1e6, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic_for(plan) if (size == SIZE and nsrc == N_SRC) else None,
                     "kernel_ms_avg": round(k_us / 1e3, 4), "launches_timed": k,
                     "kernel_ms_avg_event_pair_each": round(float(np.mean(kms)), 4),
                     "achieved_rotating_dst": round(rot, 2), "frac_rotating_dst": round(rot / HBM_PEAK_GBPS, 4),
                     "kernel_ms_avg_rotating_dst": round(rot_us / 1e3, 4),
                     "frac_of_measured_read_only": round(achieved / max(peak["read_only_GBps"],
                                                                        peak["read_only_no_residency_cap_GBps"]), 4)
                     if peak else None},
        "measured_peak": peak or None,
    }

    if not a.no_cpu:
        cb, host_slab, host_out = cpu_baseline(size, nsrc)
        out["cpu_baseline"] = cb
        # same inputs on both sides: the GPU result must equal the CPU fold bit for bit
        got = np.empty(size, dtype=np.float32)
        hip.memcpy_dtoh(got, dst)
        out["matches_cpu_oracle"] = bool(got.tobytes() == host_out.tobytes())
        del host_slab, host_out, got
    else:
        out["cpu_baseline"] = None
    mc.xccl_mem_component_free(slab, MemType.ROCM)

    if not a.no_configs:
        out["configs"] = run_configs(mc, hip)
        # 8 x 1 GiB vectors: 9 GiB per launch, 12 GiB footprint with a rotating destination
        big = 1 << 28
        st, bslab = mc.xccl_mem_component_alloc(12 * big * 4, MemType.ROCM)
        if st == Status.OK:
            for j in range(8):
                assert mc.datagen_fill(bslab + j * big * 4, big, Dt.FLOAT32, 2, j) == Status.OK
            hip.device_synchronize()
            region_gbps(mc, bslab, 8, big, 4, Dt.FLOAT32, Op.SUM, 2, rot=4)
            g, us = region_gbps(mc, bslab, 8, big, 4, Dt.FLOAT32, Op.SUM, 12, rot=4)
            out["configs"]["footprint_12GiB"] = entry(
                g, us, 9 * big * 4, workload="FLOAT32 SUM, 8 sources x 268,435,456 elements (1 GiB vectors), "
                                             "destination rotating through 4 vectors", launches_timed=12)
            mc.xccl_mem_component_free(bslab, MemType.ROCM)

    if not a.no_latency:
        lat, lbuf = latency_sweep(mc, hip, a.latency_iters, a.latency_quick)
        lat.update(latency_extras(mc, hip, lbuf, min(a.latency_iters, 4000)))
        lbuf.close()
        lat["runtime_queue_rings_in_device_memory"] = latency_with_runtime_queues_in_device_memory(
            min(a.latency_iters, 4000))
        out["latency_us"] = lat
        out["mid_sizes"] = mid_sizes(mc, hip)

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
