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
  roofline         the same bytes / the kernel's average duration, measured
                   with HIP event pairs on the component's stream around each
                   launch, against 8 TB/s HBM3E
  cpu_baseline     the CPU oracle (port of the reference's host fold, one
                   thread) timed on this box on the same workload
  latency_us       small-message p50/p99 per call in us, FLOAT32 SUM, 2/4/8 sources: "sync" = the blocking
                   vtable entry, "event" = reduce_multi_nb + event_query polling (both complete through the
                   kernel's own completion word), "stream" = reduce_multi_nb + hipStreamSynchronize,
                   "graph" = single-node hipGraph launch + hipStreamSynchronize
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
N_SRC = 8
SIZE = 67108864
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "reduce_multi_f32_sum_8x256MiB_hbm_traffic.md")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--size", type=int, default=SIZE, help="elements per vector (default: the headline 67,108,864)")
    ap.add_argument("--nsrc", type=int, default=N_SRC)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-latency", action="store_true", help="skip the small-message sweep")
    ap.add_argument("--latency-iters", type=int, default=2000)
    ap.add_argument("--profile-mode", action="store_true",
                    help="for rocprofv3: only K headline launches and K launches of a 1 GiB + 1 GiB copy kernel "
                         "(the known-traffic calibration), nothing else")
    ap.add_argument("--matrix", action="store_true",
                    help="kernel GB/s of every benchmark configuration (all dtype/op pairs of the integer sweep "
                         "and the 16-source cases included); table to <out-dir>/matrix.json, nothing else")
    ap.add_argument("--replay", action="store_true",
                    help="time whole allreduce collectives of the replayed UCX call sites (8 loopback ranks on the one "
                         "GPU): blocking reductions as in the reference vs stream-ordered ones, scratch cached vs not")
    ap.add_argument("--latency-full", action="store_true",
                    help="all 14 sizes x 10,000 iterations; table to <out-dir>/latency.json")
    ap.add_argument("--out-dir", default=os.path.join(ROOT, "bench_out"), help="where --matrix / --latency-full write")
    return ap.parse_args()


def cpu_baseline(size, nsrc):
    """The oracle's single-thread fold on the same workload, host memory."""
    from oracle import pyoracle as o
    from xccl_amd.types import Dt, Op
    threads = max(1, min(16, os.cpu_count() or 1))
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
    while sum(t1) < 8.0 and len(t1) < 60:
        t1.append(run(1))
    run(threads)
    tm = []
    while sum(tm) < 4.0 and len(tm) < 10:
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
        "sample": "%d calls of the full workload (%d x %d fp32, %d B/call), median %.1f ms/call; host traffic is "
                  "3*(N-1)*size*4 B/call" % (len(t1), nsrc, size, nbytes, med1 * 1e3),
        "all_cores": {"value": round(nbytes / medm / 1e9, 3), "cores": threads, "ms_per_call": round(medm * 1e3, 2)},
        "two_source_1Mi_fp32": {"value": round(3 * n1 * 4 / medc / 1e9, 3), "cores": 1,
                                "us_per_call": round(medc * 1e6, 1)},
    }, slab, out


def latency_sweep(mc, hip, iters, full):
    from xccl_amd.types import Dt, MemType, Op, Status
    sizes_b = [4 << k for k in range(14)] if full else [4, 1024, 32768]
    if full:
        iters = 10000
    res = {}
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
                st, ns = mc.bench_latency(mode, buf.ptr, buf.ptr + maxb, buf.ptr + 9 * maxb, nsrc - 1, cnt, maxb,
                                          Dt.FLOAT32, Op.SUM, iters)
                assert st == Status.OK, (mode, st)
                ns = ns[iters // 10:]
                row[mode] = {"p50": round(float(np.percentile(ns, 50)) / 1e3, 2),
                             "p99": round(float(np.percentile(ns, 99)) / 1e3, 2)}
            res["n%d_%dB" % (nsrc, b)] = row
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
    buf.close()
    return res


def matrix(mc, hip, out_dir):
    """Event-timed kernel bandwidth of each benchmark configuration at its full size."""
    from xccl_amd.types import Dt, MemType, Op, Status, dt_size, INT_OPS
    cases = [("config1", Dt.FLOAT32, Op.SUM, 2, 1048576)]
    cases += [("config2", Dt.FLOAT32, Op.SUM, 8, 67108864)]
    for dt in (Dt.INT8, Dt.INT16, Dt.INT32, Dt.INT64, Dt.UINT32, Dt.UINT64):
        cases += [("config3", dt, op, 4, 16777216) for op in INT_OPS]
    for dt in (Dt.FLOAT16, Dt.FLOAT64):
        cases += [("config4", dt, op, 16, 33554432) for op in (Op.SUM, Op.MAX, Op.MIN)]
    cases += [("extra", Dt.FLOAT32, Op.SUM, n, 67108864) for n in (2, 3, 4, 5, 16)]
    cases += [("extra", Dt.UINT8, op, 4, 67108864) for op in (Op.SUM, Op.MAX)]
    cases += [("extra", Dt.FLOAT16, Op.PROD, 8, 67108864), ("extra", Dt.FLOAT32, Op.MAX, 8, 67108864)]
    cases += [("inplace", Dt.FLOAT32, Op.MAX, n, 67108864) for n in (4, 8)]
    # message-size sweep: where the call leaves the launch-bound regime and reaches the bandwidth plateau
    cases += [("sweep", Dt.FLOAT32, Op.SUM, n, 1 << k) for n in (2, 4, 8) for k in range(14, 27, 2)]
    rows = []
    cur = None
    for name, dt, op, nsrc, size in cases:
        es = dt_size(dt)
        stride = size * es
        key = (dt, nsrc, size, op in (Op.LAND, Op.LOR, Op.LXOR))
        if key != cur:
            if cur is not None:
                mc.xccl_mem_component_free(buf, MemType.ROCM)
            st, buf = mc.xccl_mem_component_alloc((nsrc + 1) * stride, MemType.ROCM)
            assert st == Status.OK
            for j in range(nsrc):
                assert mc.datagen_fill(buf + j * stride, size, dt, 3, j, key[3]) == Status.OK
            hip.device_synchronize()
            cur = key
        # "inplace": rbuf == sbuf1, the form every k-nomial round after the first has (allreduce_knomial.c:118-121)
        rbuf = buf if name == "inplace" else buf + nsrc * stride
        st, k = mc.bench_kernel_times(buf, buf + stride, rbuf, nsrc - 1, size, stride, dt, op, 12)
        assert st == Status.OK
        ms = float(np.mean(k[2:]))
        nb = (nsrc + 1) * size * es
        rows.append({"config": name, "dtype": dt.name, "op": op.name, "nsrc": nsrc, "size": size, "bytes": nb,
                     "kernel_ms": round(ms, 4), "GBps": round(nb / ms / 1e6, 1),
                     "frac_of_peak": round(nb / ms / 1e6 / HBM_PEAK_GBPS, 3)})
        if name == "sweep":     # what a caller of the blocking entry sees per call, host clock
            st, ns = mc.bench_latency("sync", buf, buf + stride, buf + nsrc * stride, nsrc - 1, size, stride, dt, op,
                                      200)
            assert st == Status.OK
            rows[-1]["blocking_call_us"] = round(float(np.percentile(ns[20:], 50)) / 1e3, 2)
            rows[-1]["blocking_call_GBps"] = round(nb / rows[-1]["blocking_call_us"] / 1e3, 1)
        print("%-8s %-8s %-5s N=%-2d size=%-9d %8.4f ms %8.1f GB/s %s" % (
            name, dt.name, op.name, nsrc, size, ms, rows[-1]["GBps"],
            "blocking call %.2f us" % rows[-1]["blocking_call_us"] if name == "sweep" else ""),
            file=sys.stderr, flush=True)
    mc.xccl_mem_component_free(buf, MemType.ROCM)
    os.makedirs(out_dir, exist_ok=True)
    json.dump(rows, open(os.path.join(out_dir, "matrix.json"), "w"), indent=1)
    print(json.dumps({"matrix_rows": len(rows), "min_GBps": min(r["GBps"] for r in rows if r["config"] not in ("config1", "sweep", "inplace")),
                      "file": os.path.join(out_dir, "matrix.json")}))
    return 0


def replay_bench(mc, hip, out_dir):
    """Whole-collective times of the replayed call sites.  The loopback transport moves bytes with device
    copies, so the figures show what the reduction path and the scratch allocation contribute to a
    collective, not what a network would."""
    from xccl_amd.types import Dt, MemType, Op, Status
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

    if a.matrix:
        return matrix(mc, hip, a.out_dir)
    if a.replay:
        return replay_bench(mc, hip, a.out_dir)

    size, nsrc = a.size, a.nsrc
    stride = size * 4
    nbytes = (nsrc + 1) * size * 4
    st, slab = mc.xccl_mem_component_alloc((nsrc + 1) * stride, MemType.ROCM)
    assert st == Status.OK
    dst = slab + nsrc * stride
    for j in range(nsrc):
        assert mc.datagen_fill(slab + j * stride, size, Dt.FLOAT32, 2, j) == Status.OK
    hip.device_synchronize()
    stream = mc.component_stream()

    if a.profile_mode:
        for _ in range(a.warmup + a.steps):
            st_, _ = mc.xccl_mem_component_reduce_multi_nb(slab, slab + stride, dst, nsrc - 1, size, stride,
                                                           Dt.FLOAT32, Op.SUM, MemType.ROCM, None, want_event=False)
            assert st_ == Status.OK
        hip.stream_synchronize(stream)
        gib = 1 << 30
        for _ in range(a.warmup + a.steps):     # sources 0-3 -> sources 4-7: reads 1 GiB, writes 1 GiB
            assert mc.bench_copy(slab + 4 * stride, slab, gib, stream) == Status.OK
        hip.stream_synchronize(stream)
        print(json.dumps({"profile_mode": True, "reduce_launches": a.warmup + a.steps,
                          "copy_launches": a.warmup + a.steps, "copy_bytes_read": gib, "copy_bytes_written": gib,
                          "reduce_algorithmic_bytes": nbytes}))
        return 0

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

    # the blocking vtable entry (launch + synchronize inside), for comparison
    t0 = time.perf_counter()
    for _ in range(a.steps):
        assert mc.xccl_mem_component_reduce_multi(slab, slab + stride, dst, nsrc - 1, size, stride, Dt.FLOAT32, Op.SUM,
                                                  MemType.ROCM) == Status.OK
    sync_ms = (time.perf_counter() - t0) / a.steps * 1e3

    # per-launch device time from HIP event pairs on the kernel's own stream
    st, kms = mc.bench_kernel_times(slab, slab + stride, dst, nsrc - 1, size, stride, Dt.FLOAT32, Op.SUM,
                                    max(a.steps, 10))
    assert st == Status.OK
    # ... and from one event pair around the same number of back-to-back launches: the average launch
    # duration over the region, free of the ~5 us a per-launch event pair adds
    st, region_ms = mc.bench_region_time(slab, slab + stride, dst, nsrc - 1, size, stride, Dt.FLOAT32, Op.SUM,
                                         max(a.steps, 10))
    assert st == Status.OK
    k_avg = region_ms / max(a.steps, 10)
    achieved = nbytes / (k_avg * 1e-3) / 1e9
    traffic = None
    if os.path.isfile(TRAFFIC_FILE) and size == SIZE and nsrc == N_SRC:
        # measured once with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (the file gives the commands)
        for line in open(TRAFFIC_FILE):
            if line.strip().startswith("bytes_per_launch:"):
                traffic = int(float(line.split(":")[1]))
    # Supplementary: the same call cycling through 4 destination vectors (1 GiB), so that the
    # 256 MiB destination cannot stay resident in the 256 MB Infinity Cache between launches.
    rot = None
    st_r, rslab = mc.xccl_mem_component_alloc(4 * stride, MemType.ROCM)
    if st_r == Status.OK:
        rk = []
        for r in range(3):
            for q in range(4):
                st_q, kq = mc.bench_kernel_times(slab, slab + stride, rslab + q * stride, nsrc - 1, size, stride,
                                                 Dt.FLOAT32, Op.SUM, 1)
                assert st_q == Status.OK
                if r > 0:
                    rk.append(float(kq[0]))
        rot = round(nbytes / (float(np.mean(rk)) * 1e-3) / 1e9, 2)
        mc.xccl_mem_component_free(rslab, MemType.ROCM)

    # Reference point: a plain 1 GiB -> 1 GiB copy kernel on the same slab (2 GiB of traffic per launch),
    # i.e. what a 1:1 read/write stream reaches on this box.
    copy_gbps = None
    if nsrc >= 8 and stride * 4 >= (1 << 30):
        gib = 1 << 30
        for _ in range(3):
            assert mc.bench_copy(slab + 4 * stride, slab, gib, stream) == Status.OK
        hip.stream_synchronize(stream)
        t0 = time.perf_counter()
        for _ in range(20):
            assert mc.bench_copy(slab + 4 * stride, slab, gib, stream) == Status.OK
        hip.stream_synchronize(stream)
        copy_gbps = round(2 * gib * 20 / (time.perf_counter() - t0) / 1e9, 2)
        for j in range(4, 8):                   # the copy overwrote sources 4-7: restore them
            assert mc.datagen_fill(slab + j * stride, size, Dt.FLOAT32, 2, j) == Status.OK
        hip.device_synchronize()
        assert mc.xccl_mem_component_reduce_multi(slab, slab + stride, dst, nsrc - 1, size, stride, Dt.FLOAT32, Op.SUM,
                                                  MemType.ROCM) == Status.OK

    grid, block, name = mc._c.c_uint(0), mc._c.c_uint(0), mc._c.create_string_buffer(256)
    mc.component_lib().xccl_rocm_reduce_multi_plan(slab, slab + stride, dst, nsrc - 1, size, stride, int(Dt.FLOAT32),
                                                   int(Op.SUM), mc._c.byref(grid), mc._c.byref(block), name, 256)

    out = {
        "metric": "reduce_multi GB/s (fp32 sum, %d srcs x %d MiB)" % (nsrc, stride >> 20),
        "value": round(gbps, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "reduce_multi FLOAT32 SUM, %d source vectors x %d elements at stride %d B in one slab "
                               "(radix-8 k-nomial step); stream-ordered launches" % (nsrc, size, stride),
                   "bytes_per_step": nbytes, "device": "gfx950 (%s)" % hip.device_name(0),
                   "kernel": name.value.decode(), "grid": grid.value, "block": block.value},
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "sync_entry": {"ms_per_step": round(sync_ms, 4), "GBps": round(nbytes / sync_ms / 1e6, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "kernel_ms_avg": round(k_avg, 4), "launches_timed": max(a.steps, 10),
                     "kernel_ms_avg_event_pair_each": round(float(np.mean(kms)), 4),
                     "kernel_ms_min_event_pair_each": round(float(np.min(kms)), 4), "achieved_rotating_dst": rot,
                     "copy_kernel_GBps": copy_gbps},
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

    if not a.no_latency:
        lat = latency_sweep(mc, hip, a.latency_iters, a.latency_full)
        if a.latency_full:
            os.makedirs(a.out_dir, exist_ok=True)
            json.dump(lat, open(os.path.join(a.out_dir, "latency.json"), "w"), indent=1)
            out["latency_us"] = {k: v for k, v in lat.items()
                                 if k.endswith(("_4B", "_1024B", "_32768B")) or k.startswith(("mem_type", "alloc_free", "threads", "memcpy"))}
        else:
            out["latency_us"] = lat

    mc.xccl_mem_component_free(slab, MemType.ROCM)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
