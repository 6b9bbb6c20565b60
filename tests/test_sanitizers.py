"""The host-side C of the component that runs without a device -- the
freed-block cache (mc_pool.c) and the dispatcher (mc_dispatch.c) -- under
AddressSanitizer + UndefinedBehaviorSanitizer and under ThreadSanitizer: each
is built with its test harness into a program of its own and run as a child
process (tests/san_pool_main.c, tests/san_dispatch_main.c).  Any sanitizer
report fails the test.  The stress loops are the ones the other CPU tests use
(pool_harness.c, dispatch_stress.c): 8 threads on one lock / one atomically
claimed buffer."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "xccl_amd", "csrc")
INC = os.path.join(ROOT, "include")
T = os.path.join(ROOT, "tests")
SANITIZERS = {"asan_ubsan": ["-fsanitize=address,undefined", "-fno-sanitize-recover=all"],
              "tsan": ["-fsanitize=thread"]}
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:exitcode=23", UBSAN_OPTIONS="halt_on_error=1:exitcode=23",
           TSAN_OPTIONS="halt_on_error=1:exitcode=23:second_deadlock_stack=1")
ENV.pop("LD_PRELOAD", None)      # a sanitizer runtime insists on being the first library of its process
BASE = ["gcc", "-std=gnu11", "-O1", "-g", "-fno-omit-frame-pointer", "-Wall", "-Wextra", "-Werror"]


def _runtime_works(flags, tmp_path):
    src = tmp_path / "probe.c"
    src.write_text("int main(void){return 0;}\n")
    exe = tmp_path / "probe"
    if subprocess.run(["gcc"] + flags + ["-o", str(exe), str(src)], capture_output=True).returncode != 0:
        return False
    return subprocess.run([str(exe)], env=ENV, capture_output=True).returncode == 0


def _run(cmd):
    out = subprocess.run(cmd, env=ENV, capture_output=True, text=True, timeout=600)
    report = out.stdout + out.stderr
    assert out.returncode == 0, report
    assert "Sanitizer" not in report and "runtime error" not in report, report
    return out.stdout


@pytest.mark.parametrize("san", sorted(SANITIZERS))
def test_mem_pool_under_sanitizer(san, tmp_path):
    flags = SANITIZERS[san]
    if not _runtime_works(flags, tmp_path):
        pytest.skip("gcc's %s runtime does not run here" % san)
    exe = str(tmp_path / "san_pool")
    subprocess.run(BASE + flags + ["-I", CSRC, "-o", exe, os.path.join(T, "san_pool_main.c"),
                                   os.path.join(T, "pool_harness.c"), os.path.join(CSRC, "mc_pool.c"), "-lpthread"],
                   check=True)
    assert "pool ok" in _run([exe, "8", "20000" if san == "asan_ubsan" else "6000"])


@pytest.mark.parametrize("san", sorted(SANITIZERS))
def test_dispatcher_under_sanitizer(san, tmp_path):
    flags = SANITIZERS[san]
    if not _runtime_works(flags, tmp_path):
        pytest.skip("gcc's %s runtime does not run here" % san)
    plugins = tmp_path / "plugins"
    plugins.mkdir()
    fake = os.path.join(T, "fake_component.c")
    for fname, defs in (("xccl_cuda_mem_component.so", ["-DFAKE_SYMBOL=xccl_cuda_mem_component", "-DFAKE_MEMTYPE=1"]),
                        ("xccl_rocm_mem_component.so", ["-DFAKE_SYMBOL=xccl_rocm_mem_component", "-DFAKE_MEMTYPE=3",
                                                        "-DFAKE_EXT_SYMBOL=xccl_rocm_mem_component_ext"])):
        subprocess.run(BASE + flags + ["-shared", "-fPIC", "-I", INC, "-o", str(plugins / fname), fake] + defs, check=True)
    exe = str(tmp_path / "san_dispatch")
    subprocess.run(BASE + flags + ["-I", INC, "-o", exe, os.path.join(T, "san_dispatch_main.c"),
                                   os.path.join(T, "dispatch_stress.c"), os.path.join(CSRC, "mc_dispatch.c"),
                                   "-lpthread", "-ldl"], check=True)
    assert "dispatch ok" in _run([exe, str(plugins), "8", "50000" if san == "asan_ubsan" else "10000"])
