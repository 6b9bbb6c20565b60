"""Run under a profiler by tests/test_gpu_under_profiler.py: four host threads
issue blocking reduce_multi calls at once, two of them on each of the
component's dispatch queues, often enough for each queue's packet ring to wrap
many times; checks every result and prints `ok <calls>`."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from xccl_amd import hip, mc  # noqa: E402
from xccl_amd.types import Dt, MemType, Op, Status  # noqa: E402


def main() -> int:
    threads, iters = 4, int(sys.argv[1]) if len(sys.argv) > 1 else 2000
    print("started", flush=True)
    assert mc.xccl_mem_component_init() == Status.OK
    pitch = 8192
    buf = hip.DeviceBuffer(threads * pitch)
    host = np.zeros(threads * pitch // 4, dtype=np.float32)
    for t in range(threads):
        host[t * pitch // 4: t * pitch // 4 + 1024] = np.arange(1024, dtype=np.float32) + t
    buf.upload(host)
    hip.device_synchronize()
    before = mc.component_lib().xccl_rocm_direct_launch_count()
    # per thread: sbuf1 = 256 floats at +0, three more vectors at +1024, +2048, +3072 bytes, result at +4096
    st, ns = mc.bench_latency_mt(threads, pitch, buf.ptr, buf.ptr + 1024, buf.ptr + 4096, 3, 256, 1024, Dt.FLOAT32, Op.SUM,
                                 iters)
    assert st == Status.OK, st
    launched = mc.component_lib().xccl_rocm_direct_launch_count() - before
    assert launched == threads * iters, (launched, threads * iters)
    got = buf.download(np.float32, threads * pitch // 4)
    for t in range(threads):
        v = host[t * pitch // 4: t * pitch // 4 + 1024].reshape(4, 256)
        want = ((v[0] + v[1]) + v[2]) + v[3]
        assert np.array_equal(got[t * pitch // 4 + 1024: t * pitch // 4 + 1280], want), t
    buf.close()
    mc.xccl_mem_component_finalize()
    print("ok %d" % launched)
    return 0


if __name__ == "__main__":
    sys.exit(main())
