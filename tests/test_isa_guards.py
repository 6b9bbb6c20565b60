"""Static checks on the gfx950 assembly of every reduction kernel (no GPU):
code-generation properties the design relies on and that a compiler upgrade
or an innocent-looking source edit could silently undo.  Compiles the five
kernel translation units with `hipcc -S`."""
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
    # two kernels per (type, op) family -- the walk and the burst for small launches -- each for any number of sources
    counts = {u: len(_kernels(t)) for u, t in asm.items()}
    assert counts == {"reduce_w8": 24, "reduce_w16": 18, "reduce_w32": 18, "reduce_w64": 18, "reduce_fp": 24}
    for t in asm.values():
        names = list(_kernels(t))
        assert sum(_is_burst(n) for n in names) * 2 == len(names)


def _is_burst(name):
    """reduce_multi_kernel<T, Op, true>: the last template argument is mangled as Lb1E."""
    assert "Lb0EEEv" in name or "Lb1EEEv" in name, name
    return "Lb1EEEv" in name


def _instructions(body):
    return [ln.strip() for ln in body.splitlines() if ln.startswith("\t") and not ln.strip().startswith((".", ";"))]


def test_completion_word_waits_for_the_result_stores(asm):
    """The wave that counts itself into the completion word must first wait
    for its own write-through stores: an explicit `s_waitcnt vmcnt(0)` (the
    only inline-asm statement of the kernels) lies behind every vector store
    and ahead of every arrival atomic and of the store that publishes the
    sequence number.  Without it the host can see the word before the data."""
    for u, text in asm.items():
        for name, body in _kernels(text).items():
            blocks = re.findall(r";;#ASMSTART\n(.*?);;#ASMEND", body, flags=re.S)
            assert [b.strip() for b in blocks] == ["s_waitcnt vmcnt(0)"], (name, blocks)
            wait = body.index(";;#ASMSTART")
            stores = [m.start() for m in re.finditer(r"\bbuffer_store_\w+\b", body)]
            atomics = [m.start() for m in re.finditer(r"\bglobal_atomic_inc\b", body)]
            publish = [m.start() for m in re.finditer(r"\bglobal_store_dword\b[^\n]* sc0 sc1", body)]
            # two publishing stores: one word per workgroup for a handful of workgroups, the counted path's last arriver
            assert stores and len(atomics) == 2 and len(publish) == 2, (name, len(stores), len(atomics), len(publish))
            assert max(stores) < wait < min(atomics + publish), name
            # nothing branches from the tile loop to behind the wait: the label the loop exits to precedes it
            assert not re.search(r"\bbuffer_(load|store)_\w+\b", body[wait:]), name
            # every result store is a buffer store with write-through policy: the publishing stores (system-scope
            # releases, which bring the kernel's only cache write-backs) are the only global/flat stores
            assert len(re.findall(r"\b(global|flat)_store_\w+", body)) == 2, name
            assert body.count("buffer_wbl2") == 2, name


def test_code_generation_properties(asm):
    for u, text in asm.items():
        for name, body in _kernels(text).items():
            # no register spilling to scratch memory: the kernels are HBM streams, a spill doubles traffic
            assert re.search(r"\.amdhsa_private_segment_fixed_size 0\b", body), name
            # packed-fp32 arithmetic is compiled out (the build passes -packed-fp32-ops)
            assert not re.search(r"\bv_pk_(add|mul|fma)_f32\b", body), name
            # the tile path moves 16 bytes per lane per access through buffer instructions whose
            # cache-policy bits the compiler sees: non-temporal loads, system-scope write-through stores
            ins = _instructions(body)
            loads = [i for i in ins if i.startswith("buffer_load_")]
            stores = [i for i in ins if i.startswith("buffer_store_")]
            assert any(i.startswith("buffer_load_dwordx4") for i in loads) and all(i.endswith(" nt") for i in loads), name
            assert any(i.startswith("buffer_store_dwordx4") for i in stores) and \
                all(i.endswith(" sc0 sc1") for i in stores), name
            # head and tail elements take the same route: no global/flat loads of operands at all
            assert not re.search(r"\b(global|flat)_load_(u?byte|u?short|dword)", body), name
            # the kernel argument block is ReduceArgs and nothing else (no implicit launch arguments): the
            # component's own dispatch queue passes exactly that
            assert re.search(r"\.amdhsa_kernarg_size 96\b", body), name
            # few registers: 24 or more waves fit a compute unit
            assert int(re.search(r"\.amdhsa_next_free_vgpr (\d+)", body).group(1)) <= 80, name


def test_sources_are_walked_with_two_loads_in_flight(asm):
    """The walk through the sources keeps its issue order: never more than
    three vector loads without a wait between them (sbuf1 and the first two
    vectors of sbuf2 at the start, one at a time afterwards), and the loop
    waits with one load still in flight (vmcnt(1)), not for all of them."""
    for u, text in asm.items():
        for name, body in _kernels(text).items():
            if _is_burst(name):
                continue
            run = longest = 0
            for i in _instructions(body):
                if i.startswith("buffer_load_dwordx4"):
                    run += 1
                    longest = max(longest, run)
                elif i.startswith("s_waitcnt") and "vmcnt" in i:
                    run = 0
            assert longest <= 3, (name, longest)
            assert "s_waitcnt vmcnt(1)" in body, name


def test_burst_kernels_issue_every_load_of_a_tile_at_once(asm):
    """The kernels for small launches ask for sbuf1 and eight vectors of sbuf2
    before they wait for any of them, and then fold them as they arrive."""
    for u, text in asm.items():
        for name, body in _kernels(text).items():
            if not _is_burst(name):
                continue
            run = longest = 0
            for i in _instructions(body):
                if i.startswith("buffer_load_dwordx4"):
                    run += 1
                    longest = max(longest, run)
                elif i.startswith("s_waitcnt") and "vmcnt" in i:
                    run = 0
            assert longest >= 8, (name, longest)     # the compiler may start folding before the ninth


def test_float_min_max_stay_compare_select(asm):
    """`a > b ? a : b` must not become v_max/v_min: those order signed zeros
    and propagate NaN differently from the ternary of the reference."""
    for name, body in _kernels(asm["reduce_fp"]).items():
        if "OpMax" in name or "OpMin" in name:
            assert not re.search(r"\bv_(pk_)?(max|min)(imum)?(_num)?_f(16|32|64)\b", body), name
            assert re.search(r"\bv_cmp_(gt|lt|ngt|nlt|ge|le|nge|nle)_f(16|32|64)", body) or \
                re.search(r"\bv_cmp\w*_f(16|32|64)", body), name
