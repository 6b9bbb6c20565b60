"""The component's own dispatch queues under a tool that interposes on queue
submission.  rocprofv3 replaces every HSA queue by an intercept queue whose
handler copies the packets that are new at a doorbell; when two threads shared
one of the component's queues and both had a packet pending across the ring's
wrap, that handler read past the end of the ring (a host segmentation fault at
exactly base + 256 packets).  Submission is now one producer at a time per
queue, so every doorbell stands for one new packet.  This runs the four-thread
case under the profiler, in a child process."""
import csv
import glob
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MAIN = os.path.join(ROOT, "tests", "profiled_threads_main.py")


@pytest.mark.gpu
def test_four_threads_on_two_shared_queues_under_rocprofv3(tmp_path):
    prof = shutil.which("rocprofv3")
    if prof is None:
        pytest.skip("rocprofv3 is not on PATH")
    iters = 2000                     # 4000 packets per queue: each 256-packet ring wraps 15 times
    out = tmp_path / "trace"
    env = dict(os.environ, TMPDIR=str(tmp_path))
    res = subprocess.run([prof, "--kernel-trace", "--output-format", "csv", "-d", str(out), "--", sys.executable, MAIN,
                          str(iters)], cwd=str(tmp_path), env=env, capture_output=True, text=True, timeout=110)
    tail = (res.stdout + res.stderr)[-1500:]
    if "started" not in res.stdout:
        pytest.skip("rocprofv3 did not get as far as starting the program here: " + tail[-300:])
    assert res.returncode == 0, tail
    assert "ok %d" % (4 * iters) in res.stdout, tail
    traces = glob.glob(str(out / "**" / "*_kernel_trace.csv"), recursive=True)
    assert traces, tail
    rows = sum(1 for f in traces for r in csv.DictReader(open(f)) if "reduce_multi_kernel" in r["Kernel_Name"])
    assert rows >= 4 * iters, rows   # the profiler saw every launch
