"""integration/xccl-rocm.patch -- the edits to the reference tree that make
libxccl load and use the ROCm memory component -- must apply to the reference
as it is, and the patched files must compile: checked on a scratch copy, with
a compiler run over every file the patch touches and over the component built
the in-tree way (-DXCCL_MC_ROCM_IN_TREE) against the patched headers.  UCX is
not installed here; tests/stubs holds declarations of the few UCX types and
calls those files name.  Skipped where the reference tree is not present."""
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


# ---- a compiler over the patched tree ----------------------------------------

STUBS = os.path.join(ROOT, "tests", "stubs")
CSRC = os.path.join(ROOT, "xccl_amd", "csrc")
# mistakes a patch can introduce and plain C lets through as warnings
STRICT = ["-Werror=implicit-function-declaration", "-Werror=incompatible-pointer-types", "-Werror=int-conversion",
          "-Werror=implicit-int", "-Werror=return-type"]
COMPILED = ("src/utils/mem_component.c", "src/team_lib/ucx/xccl_ucx_lib.c",
            "src/team_lib/ucx/allreduce/allreduce_knomial.c", "src/team_lib/ucx/allreduce/allreduce_sra.c",
            "src/team_lib/ucx/reduce/reduce_knomial.c", "src/team_lib/ucx/reduce/reduce_linear.c")


@pytest.fixture(scope="module")
def patched_tree(tmp_path_factory):
    if not os.path.isdir(REFERENCE):
        pytest.skip("reference tree not present")
    d = tmp_path_factory.mktemp("patched")
    shutil.copytree(os.path.join(REFERENCE, "src"), d / "src")
    subprocess.run(["patch", "-s", "-p1", "--fuzz=0", "-i", PATCH], cwd=d, check=True)
    return d


def _tree_includes(tree):
    return ["-I", STUBS, "-I", str(tree / "src"), "-I", str(tree / "src/core"), "-I", str(tree / "src/utils"),
            "-I", str(tree / "src/team_lib/ucx")]


def _cc(args):
    out = subprocess.run(["gcc", "-std=gnu11", "-O1", "-c", "-o", os.devnull] + STRICT + args, capture_output=True,
                         text=True)
    assert out.returncode == 0, " ".join(args) + "\n" + out.stderr


@pytest.mark.parametrize("source", COMPILED)
def test_patched_reference_file_compiles(patched_tree, source):
    """The dispatcher, the team library's gating file and the four call-site
    files (reference src/utils/mem_component.c:30,176-178,
    xccl_ucx_lib.c:639-640, allreduce_knomial.c:74-80,129-135,
    allreduce_sra.c:212-218,281-284, reduce_knomial.c:79-85,
    reduce_linear.c:28-34) after the patch."""
    _cc(_tree_includes(patched_tree) + [str(patched_tree / source)])


@pytest.mark.parametrize("source", COMPILED)
def test_stubs_also_carry_the_unpatched_file(source):
    """The same stand-in headers compile the files as they lie in the reference
    tree: what the patched build shows is about the patch, not the stubs."""
    if not os.path.isdir(REFERENCE):
        pytest.skip("reference tree not present")
    from pathlib import Path
    _cc(_tree_includes(Path(REFERENCE)) + [os.path.join(REFERENCE, source)])


@pytest.mark.parametrize("source", ("mc_rocm.c", "mc_dispatch.c", "ucx_replay.c"))
def test_component_compiles_in_tree(patched_tree, source):
    """The in-tree build of the component: types, vtable and dispatcher
    declarations come from the patched tree's own headers, so a signature that
    differs between include/xccl_rocm_mem_component.h and the patch's
    src/utils/mem_component.h is a `conflicting types` error here.
    mc_dispatch.c and ucx_replay.c are never part of an in-tree build (libxccl
    has its own dispatcher and call sites); compiling them this way checks
    that the stand-in dispatcher DEFINES, and the replayed call sites CALL,
    every entry exactly as the patched header declares it."""
    _cc(["-DXCCL_MC_ROCM_IN_TREE", "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include", "-I",
         os.path.join(ROOT, "include")] + _tree_includes(patched_tree) + [os.path.join(CSRC, source)])


def test_in_tree_build_catches_a_signature_mismatch(patched_tree, tmp_path):
    """The check above has teeth: dropping the stream argument from the patched
    header's declaration makes the component's build fail."""
    hdr = patched_tree / "src/utils/mem_component.h"
    text = hdr.read_text()
    broken = text.replace("xccl_stream_t *stream,\n                                           xccl_mc_event_t **event);",
                          "xccl_mc_event_t **event);", 1)
    assert broken != text
    alt = tmp_path / "src"
    shutil.copytree(patched_tree / "src", alt)
    (alt / "utils/mem_component.h").write_text(broken)
    out = subprocess.run(["gcc", "-std=gnu11", "-fsyntax-only", "-DXCCL_MC_ROCM_IN_TREE", "-D__HIP_PLATFORM_AMD__",
                          "-I", "/opt/rocm/include", "-I", os.path.join(ROOT, "include")] + _tree_includes(tmp_path) +
                         [os.path.join(CSRC, "mc_dispatch.c")], capture_output=True, text=True)
    assert out.returncode != 0 and "conflicting types" in out.stderr
