"""integration/xccl-rocm.patch -- the edits to the reference tree that make
libxccl load and use the ROCm memory component -- must apply to the reference
as it is: checked on a scratch copy of the files it touches.  Skipped where
the reference tree is not present."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PATCH = os.path.join(ROOT, "integration", "xccl-rocm.patch")
REFERENCE = "/root/reference"

TOUCHED = ("src/api/xccl.h", "src/utils/mem_component.h", "src/utils/mem_component.c",
           "src/team_lib/ucx/xccl_ucx_lib.c", "src/team_lib/ucx/xccl_ucx_lib.h",
           "src/team_lib/ucx/allreduce/allreduce_knomial.h", "src/team_lib/ucx/allreduce/allreduce_knomial.c",
           "src/team_lib/ucx/allreduce/allreduce_sra.c", "src/team_lib/ucx/reduce/reduce_knomial.c",
           "src/team_lib/ucx/reduce/reduce_linear.c")


def test_patch_names_exactly_the_files_it_should():
    files = re.findall(r"^\+\+\+ b/(\S+)", open(PATCH).read(), flags=re.M)
    assert sorted(files) == sorted(TOUCHED)


@pytest.fixture()
def scratch_copy(tmp_path):
    if not os.path.isdir(REFERENCE):
        pytest.skip("reference tree not present")
    for f in TOUCHED:
        dst = tmp_path / f
        dst.parent.mkdir(parents=True, exist_ok=True)
        shutil.copyfile(os.path.join(REFERENCE, f), dst)
    return tmp_path


def test_patch_applies_to_the_reference_tree(scratch_copy):
    dry = subprocess.run(["patch", "-p1", "--dry-run", "--fuzz=0", "-i", PATCH], cwd=scratch_copy, capture_output=True,
                         text=True)
    assert dry.returncode == 0, dry.stdout + dry.stderr
    assert "FAILED" not in dry.stdout and "fuzz" not in dry.stdout and "offset" not in dry.stdout, dry.stdout
    real = subprocess.run(["patch", "-p1", "--fuzz=0", "-i", PATCH], cwd=scratch_copy, capture_output=True, text=True)
    assert real.returncode == 0, real.stdout + real.stderr

    def text(f):
        return open(scratch_copy / f).read()

    # gating: the three places that made a ROCm pointer XCCL_ERR_UNSUPPORTED
    assert "XCCL_STREAM_TYPE_ROCM" in text("src/api/xccl.h")
    mc = text("src/utils/mem_component.c")
    assert "[XCCL_STREAM_TYPE_ROCM] = UCS_MEMORY_TYPE_ROCM" in mc
    assert 'snprintf(sym, sizeof(sym), "xccl_%s_mem_component"' in mc and '"xccl_cuda_mem_component"' in mc
    assert "UCS_BIT(UCS_MEMORY_TYPE_ROCM)" in text("src/team_lib/ucx/xccl_ucx_lib.c")
    # call sites: every blocking reduction of the four algorithms became a stream-ordered one with a saved phase
    for f, calls in (("src/team_lib/ucx/allreduce/allreduce_knomial.c", 2), ("src/team_lib/ucx/allreduce/allreduce_sra.c", 2),
                     ("src/team_lib/ucx/reduce/reduce_knomial.c", 1), ("src/team_lib/ucx/reduce/reduce_linear.c", 1)):
        t = text(f)
        assert len(re.findall(r"xccl_mem_component_reduce(_multi)?_nb\(", t)) == calls, f
        assert not re.search(r"xccl_mem_component_reduce(_multi)?\(", t), f
        assert len(re.findall(r"xccl_ucx_reduce_test\(req\)", t)) == calls, f
        assert t.count("{") == t.count("}") and t.count("(") == t.count(")"), f
    for f in ("src/team_lib/ucx/allreduce/allreduce_knomial.c", "src/team_lib/ucx/allreduce/allreduce_sra.c"):
        t = text(f)
        for label in ("PHASE_EXTRA_REDUCE", "PHASE_1_REDUCE"):
            assert re.search(r"^\s*%s:" % label, t, flags=re.M) and "SAVE_STATE(%s)" % label in t, (f, label)
        assert "GOTO_PHASE_REDUCE(" in t
    hdr = text("src/team_lib/ucx/allreduce/allreduce_knomial.h")
    assert "PHASE_EXTRA_REDUCE," in hdr and "PHASE_1_REDUCE," in hdr and "define GOTO_PHASE_REDUCE" in hdr
    # the extension struct the dispatcher reads must agree with the component's exported object
    ext = re.search(r"typedef struct xccl_mem_component_ext \{(.*?)\} xccl_mem_component_ext_t;",
                    text("src/utils/mem_component.h"), flags=re.S).group(1)
    ours = re.search(r"typedef struct xccl_rocm_mem_component \{(.*?)\} xccl_rocm_mem_component_t;",
                     open(os.path.join(ROOT, "include", "xccl_rocm_mem_component.h")).read(), flags=re.S).group(1)

    def members(body):
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        return re.findall(r"\(\*(\w+)\)|\b(super|ext_version)\s*;", body)

    assert members(ext) == members(ours)


def test_git_apply_check(scratch_copy):
    out = subprocess.run(["git", "apply", "--check", PATCH], cwd=scratch_copy, capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
