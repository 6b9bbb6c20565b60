"""Static checks on the gfx950 assembly of every reduction kernel (no GPU):
the one inline-asm statement in the kernels is invisible to the compiler's
hazard recogniser, so the properties that keep it hazard-free are asserted on
the generated code, together with a few code-generation properties the design
relies on.  Compiles the five kernel translation units with `hipcc -S`."""
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "xccl_amd", "csrc")
UNITS = ("reduce_w8", "reduce_w16", "reduce_w32", "reduce_w64", "reduce_fp")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"), "-S",
         "--cuda-device-only"]


@pytest.fixture(scope="module")
def asm(tmp_path_factory):
    out = tmp_path_factory.mktemp("isa")

    def one(u):
        dst = os.path.join(str(out), u + ".s")
        subprocess.run(["hipcc"] + FLAGS + [os.path.join(CSRC, u + ".hip"), "-o", dst], check=True,
                       stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        return u, open(dst).read()

    with ThreadPoolExecutor(max_workers=5) as ex:
        return dict(ex.map(one, UNITS))


def _kernels(text):
    """name -> body for every reduce_multi_kernel instantiation of a unit."""
    out = {}
    for m in re.finditer(r"^(_ZN9xccl_rocm19reduce_multi_kernel\w+):.*?\n(.*?)\.end_amdhsa_kernel", text, flags=re.S | re.M):
        out[m.group(1)] = m.group(2)
    return out


def test_every_variant_is_instantiated(asm):
    # per (type, op) family: 6 source-count variants x 2 cache policies
    counts = {u: len(_kernels(t)) for u, t in asm.items()}
    assert counts == {"reduce_w8": 12 * 12, "reduce_w16": 9 * 12, "reduce_w32": 9 * 12, "reduce_w64": 9 * 12,
                      "reduce_fp": 12 * 12}


def test_asm_store_is_hazard_free_by_construction(asm):
    """(1) address in a VGPR pair with `off`, never a scalar base: a VMEM
    instruction reading an SGPR within 5 wait states of a VALU write to it
    (e.g. v_readlane restoring a spilled SGPR) sees the old value;
    (2) followed by s_nop >= 1: the data registers of a >8-byte store are read
    a cycle after issue and must not be overwritten in the next slot."""
    n = 0
    for u, text in asm.items():
        for block in re.findall(r";;#ASMSTART\n(.*?);;#ASMEND", text, flags=re.S):
            lines = [ln.strip() for ln in block.strip().splitlines()]
            if not lines:
                continue            # the empty statement that pins the completion-word pointer into SGPRs early
            assert len(lines) == 2, (u, lines)
            assert re.fullmatch(r"global_store_dwordx4 v\[\d+:\d+\], v\[\d+:\d+\], off sc0 sc1", lines[0]), (u, lines[0])
            m = re.fullmatch(r"s_nop (\d+)", lines[1])
            assert m and int(m.group(1)) >= 1, (u, lines[1])
            n += 1
    assert n > 1000


def test_code_generation_properties(asm):
    for u, text in asm.items():
        for name, body in _kernels(text).items():
            # no register spilling to scratch memory: the kernels are HBM streams, a spill doubles traffic
            assert re.search(r"\.amdhsa_private_segment_fixed_size 0\b", body), name
            # packed-fp32 arithmetic is compiled out (the build passes -packed-fp32-ops)
            assert not re.search(r"\bv_pk_(add|mul|fma)_f32\b", body), name
            # the tile path moves 16 bytes per lane per access
            assert "global_load_dwordx4" in body, name
            stream = name.endswith("Li1EEEvNS_10ReduceArgsE")
            if stream:
                assert re.search(r"global_load_dwordx4 .* nt\b", body), name
                assert re.search(r"global_store_dwordx4 .* sc0 sc1", body), name
            else:
                assert "global_store_dwordx4" in body, name
                assert not re.search(r"global_store_dwordx4 .* sc0 sc1", body), name


def test_float_min_max_stay_compare_select(asm):
    """`a > b ? a : b` must not become v_max/v_min: those order signed zeros
    and propagate NaN differently from the ternary of the reference."""
    for name, body in _kernels(asm["reduce_fp"]).items():
        if "OpMax" in name or "OpMin" in name:
            assert not re.search(r"\bv_(pk_)?(max|min)(imum)?(_num)?_f(16|32|64)\b", body), name
            assert re.search(r"\bv_cmp_(gt|lt|ngt|nlt|ge|le|nge|nle)_f(16|32|64)", body) or \
                re.search(r"\bv_cmp\w*_f(16|32|64)", body), name
