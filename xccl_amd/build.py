"""Builds the package's shared objects for gfx950 with hipcc/gcc (no GPU needed)."""
import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")

LIBS = ("xccl_rocm_mem_component.so", "libxccl_mc.so", "libxccl_rocm_benchkit.so", "libxccl_ucx_replay.so",
        "test_rocm_allreduce")


def built() -> bool:
    return all(os.path.isfile(os.path.join(LIB_DIR, n)) for n in LIBS)


def build(force: bool = True, jobs: int = 8) -> None:
    """Runs csrc/Makefile.  force=True recompiles everything (make -B)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = ["make", "-C", CSRC_DIR, "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True)
    if not built():
        raise RuntimeError("xccl_amd build did not produce %s" % (LIBS,))


if __name__ == "__main__":
    build()
