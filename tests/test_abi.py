"""Boundary checks that need no GPU: the libraries load, export every symbol
the headers declare, the exported vtable has the reference's shape, enum values
match the reference, and the dispatcher's host-side logic (loader, buffer
cache, memtype probing, forwarding, error codes) behaves like reference
src/utils/mem_component.c -- driven through a host-memory stand-in component."""
import ctypes
import os
import re
import subprocess

import pytest

from xccl_amd import mc
from xccl_amd.build import LIB_DIR
from xccl_amd.types import Dt, MemType, Op, Status, StreamType, dt_size, supported_pairs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")
REF = "/root/reference"


def _declared_functions(header):
    text = open(os.path.join(INC, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(xccl_[a-z0-9_]+)\s*\(", text)
    return sorted({n for n in names if n != "xccl_dt_size" and not n.endswith("_t")})


def test_kernel_abi_symbols_exported():
    lib = mc.component_lib()
    names = _declared_functions("xccl_rocm_kernels.h")
    assert "xccl_rocm_reduce_multi_impl" in names and len(names) >= 8
    for n in names:
        assert hasattr(lib, n), "xccl_rocm_mem_component.so does not export %s" % n


def test_dispatcher_abi_symbols_exported():
    lib = mc.dispatch_lib()
    names = [n for n in _declared_functions("xccl_rocm_mem_component.h")]
    assert "xccl_mem_component_reduce_multi" in names and len(names) >= 18
    for n in names:
        assert hasattr(lib, n), "libxccl_mc.so does not export %s" % n


def test_mem_pool_abi_symbols_exported():
    lib = mc.component_lib()
    names = _declared_functions("xccl_rocm_mem_pool.h")
    assert names == ["xccl_rocm_mem_pool_get_stats", "xccl_rocm_mem_pool_set_limit"]
    for n in names:
        assert hasattr(lib, n), "xccl_rocm_mem_component.so does not export %s" % n
    assert ctypes.sizeof(mc.MemPoolStats) == 48


def test_component_object_and_alias():
    """One object, two names: the reference loader dlsym()s
    "xccl_cuda_mem_component" for every memory type (mem_component.c:30)."""
    lib = mc.component_lib()
    a = mc.RocmMemComponent.in_dll(lib, "xccl_rocm_mem_component")
    b = mc.RocmMemComponent.in_dll(lib, "xccl_cuda_mem_component")
    assert ctypes.addressof(a) == ctypes.addressof(b)
    vt = a.super
    for name, _ in mc.MemComponentVtable._fields_[:13]:
        assert ctypes.cast(getattr(vt, name), ctypes.c_void_p).value, "vtable slot %s is NULL" % name
    assert a.ext_version == 1
    ext = ctypes.c_void_p.in_dll(lib, "xccl_rocm_mem_component_ext")      # how loaders find the extension
    assert ext.value == ctypes.addressof(a)
    for name in ("reduce_nb", "reduce_multi_nb", "event_wait", "get_stream"):
        assert ctypes.cast(getattr(a, name), ctypes.c_void_p).value
    # 13 function pointers, dlhandle, {buf,size,used(+pad)} on LP64
    assert ctypes.sizeof(mc.MemComponentVtable) == 13 * 8 + 8 + 24
    assert mc.MemComponentVtable.cache.offset == 14 * 8


def test_open_touches_no_device():
    """open() runs inside libxccl's ELF constructor; it must succeed on a
    machine state where no device has been selected (or exists)."""
    assert mc.component().super.open() == Status.OK


def test_supported_matrix():
    lib = mc.component_lib()
    ok = set(supported_pairs())
    assert len(ok) == 8 * 10 + 3 * 4
    for dt in Dt:
        for op in Op:
            st = lib.xccl_rocm_reduce_supported(int(dt), int(op))
            assert st == (Status.OK if (dt, op) in ok else Status.ERR_UNSUPPORTED), (dt, op)
    assert lib.xccl_rocm_reduce_supported(99, 2) == Status.ERR_UNSUPPORTED
    assert lib.xccl_rocm_reduce_supported(-1, 2) == Status.ERR_UNSUPPORTED


def _header_enum(text, typename):
    body = re.search(r"typedef enum[^{]*\{([^}]*)\}\s*" + typename + r"\s*;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    out, nxt = {}, 0
    for item in body.split(","):
        item = item.strip()
        if not item:
            continue
        if "=" in item:
            k, v = [s.strip() for s in item.split("=")]
            nxt = int(v, 0)
        else:
            k = item
        out[k] = nxt
        nxt += 1
    return out


def test_enum_values_match_python_mirror():
    text = open(os.path.join(INC, "xccl_rocm_types.h")).read()
    for typename, prefix, py in (("xccl_op_t", "XCCL_OP_", Op), ("xccl_dt_t", "XCCL_DT_", Dt),
                                 ("xccl_status_t", "XCCL_", Status)):
        vals = _header_enum(text, typename)
        for k, v in vals.items():
            assert py[k[len(prefix):]] == v
        assert len(vals) == len(py)
    mt = _header_enum(text, "ucs_memory_type_t")
    assert mt == {"UCS_MEMORY_TYPE_" + m.name: m.value for m in MemType}


@pytest.mark.skipif(not os.path.isdir(REF), reason="reference tree not present")
def test_enum_values_match_reference_headers():
    """Numeric values are ABI: compare with reference src/api/xccl.h:371-407 and
    src/api/xccl_status.h:10-30, read as text."""
    ours = open(os.path.join(INC, "xccl_rocm_types.h")).read()
    ref_api = open(os.path.join(REF, "src/api/xccl.h")).read()
    ref_st = open(os.path.join(REF, "src/api/xccl_status.h")).read()
    assert _header_enum(ours, "xccl_op_t") == _header_enum(ref_api, "xccl_op_t")
    assert _header_enum(ours, "xccl_dt_t") == _header_enum(ref_api, "xccl_dt_t")
    assert _header_enum(ours, "xccl_status_t") == _header_enum(ref_st, "xccl_status_t")
    ref_stream = _header_enum(ref_api, "xccl_stream_type_t")
    mine = _header_enum(ours, "xccl_stream_type_t")
    assert all(mine[k] == v for k, v in ref_stream.items())
    # vtable member order, reference src/utils/mem_component.h:28-49
    ref_mc = open(os.path.join(REF, "src/utils/mem_component.h")).read()
    body = re.search(r"typedef struct xccl_mem_component \{(.*?)\} xccl_mem_component_t;", ref_mc, flags=re.S).group(1)
    ref_members = re.findall(r"\(\*([a-z_]+)\)", body) + ["dlhandle", "cache"]
    assert [n for n, _ in mc.MemComponentVtable._fields_] == ref_members


def test_plan_rejects_bad_arguments_without_a_device():
    """Argument checks come before any device query: NULL operands, a vector
    count beyond 32 bits and an element count whose byte size would wrap are
    XCCL_ERR_INVALID_PARAM, an unsupported pair XCCL_ERR_UNSUPPORTED."""
    lib = mc.component_lib()
    plan = lib.xccl_rocm_reduce_multi_plan
    plan.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_size_t] * 3 + [ctypes.c_int] * 2 + [ctypes.c_void_p] * 3 + \
                    [ctypes.c_size_t]
    ok = (0x1000, 0x2000, 0x3000)
    assert plan(None, ok[1], ok[2], 1, 16, 64, int(Dt.INT32), int(Op.SUM), None, None, None, 0) == Status.ERR_INVALID_PARAM
    assert plan(ok[0], None, ok[2], 1, 16, 64, int(Dt.INT32), int(Op.SUM), None, None, None, 0) == Status.ERR_INVALID_PARAM
    assert plan(ok[0], ok[1], None, 1, 16, 64, int(Dt.INT32), int(Op.SUM), None, None, None, 0) == Status.ERR_INVALID_PARAM
    assert plan(*ok, 1 << 32, 16, 64, int(Dt.INT32), int(Op.SUM), None, None, None, 0) == Status.ERR_INVALID_PARAM
    assert plan(*ok, 1, (1 << 56) + 1, 64, int(Dt.INT32), int(Op.SUM), None, None, None, 0) == Status.ERR_INVALID_PARAM
    assert plan(*ok, 1, 16, 64, int(Dt.FLOAT32), int(Op.BAND), None, None, None, 0) == Status.ERR_UNSUPPORTED
    assert plan(*ok, 1, 16, 64, int(Dt.INT128), int(Op.SUM), None, None, None, 0) == Status.ERR_UNSUPPORTED


def test_dt_size():
    assert [dt_size(d) for d in (Dt.INT8, Dt.INT16, Dt.INT32, Dt.INT64, Dt.INT128, Dt.UINT8, Dt.UINT16, Dt.UINT32,
                                 Dt.UINT64, Dt.UINT128, Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64, Dt.LAST_PREDEFINED,
                                 Dt.UNSUPPORTED)] == [1, 2, 4, 8, 16, 1, 2, 4, 8, 16, 2, 4, 8, 0, 0]


# ---- dispatcher logic through a stand-in component ---------------------------

@pytest.fixture(scope="module")
def fake(tmp_path_factory):
    """Builds tests/fake_component.c as xccl_cuda_mem_component.so (exports the
    hard-coded name, plain reference vtable) and
    xccl_cuda-managed_mem_component.so (exports its own name only, and the
    stream-ordered extension under xccl_cuda_managed_mem_component_ext), and
    loads them through xccl_mem_component_init."""
    d = tmp_path_factory.mktemp("plugins")
    src = os.path.join(ROOT, "tests", "fake_component.c")
    libs = {}
    for fname, sym, mt in (("xccl_cuda_mem_component.so", "xccl_cuda_mem_component", MemType.CUDA),
                           ("xccl_cuda-managed_mem_component.so", "xccl_cuda_managed_mem_component",
                            MemType.CUDA_MANAGED)):
        out = os.path.join(str(d), fname)
        ext = ["-DFAKE_EXT_SYMBOL=%s_ext" % sym] if mt == MemType.CUDA_MANAGED else []
        subprocess.run(["gcc", "-shared", "-fPIC", "-O1", "-Wall", "-Werror", "-I", INC, "-DFAKE_SYMBOL=" + sym,
                        "-DFAKE_MEMTYPE=%d" % int(mt), "-o", out, src] + ext, check=True)
        libs[mt] = ctypes.CDLL(out)
    # a file that exports neither name must be skipped, not dereferenced
    bad = os.path.join(str(d), "xccl_rocm-managed_mem_component.so")
    subprocess.run(["gcc", "-shared", "-fPIC", "-x", "c", "-o", bad, "-"], input=b"int unrelated;", check=True)
    os.environ["XCCL_MEM_COMPONENT_CACHE_SIZE"] = "4096"
    assert mc.xccl_mem_component_init(str(d)) == Status.OK
    return libs


def _calls(lib):
    return list((ctypes.c_int * 16).in_dll(lib, "fake_calls"))


def test_loader_finds_both_symbol_names_and_skips_bad_file(fake):
    get = mc.dispatch_lib().xccl_mem_component_get
    assert bool(get(int(MemType.CUDA))) and bool(get(int(MemType.CUDA_MANAGED)))
    assert not bool(get(int(MemType.ROCM_MANAGED)))
    assert not bool(get(int(MemType.HOST))) and not bool(get(17)) and not bool(get(-1))
    vt = get(int(MemType.CUDA)).contents
    assert vt.cache.size == 4096 and vt.cache.used == 0 and not vt.cache.buf and vt.dlhandle
    assert _calls(fake[MemType.CUDA])[0] == 1  # open() once


def test_alloc_cache_semantics(fake):
    """mem_component.c:51-105: one cached buffer of cache.size bytes, lent when
    idle and big enough; freeing it only clears `used`."""
    lib = fake[MemType.CUDA]
    n0 = _calls(lib)
    st, p1 = mc.xccl_mem_component_alloc(100, MemType.CUDA)
    assert st == Status.OK and p1
    vt = mc.dispatch_lib().xccl_mem_component_get(int(MemType.CUDA)).contents
    assert vt.cache.buf == p1 and vt.cache.used == 1
    assert _calls(lib)[1] == n0[1] + 1          # allocated cache.size once
    st, p2 = mc.xccl_mem_component_alloc(100, MemType.CUDA)   # cache busy -> real allocation
    assert st == Status.OK and p2 != p1 and _calls(lib)[1] == n0[1] + 2
    assert mc.xccl_mem_component_free(p1, MemType.CUDA) == Status.OK
    assert vt.cache.used == 0 and _calls(lib)[2] == n0[2]      # no mem_free for the cached buffer
    st, p3 = mc.xccl_mem_component_alloc(4096, MemType.CUDA)   # fits exactly -> cached buffer again, no alloc
    assert p3 == p1 and _calls(lib)[1] == n0[1] + 2
    assert mc.xccl_mem_component_free(p3, MemType.CUDA) == Status.OK
    st, p4 = mc.xccl_mem_component_alloc(4097, MemType.CUDA)   # too big for the cache
    assert p4 != p1 and _calls(lib)[1] == n0[1] + 3 and vt.cache.used == 0
    assert mc.xccl_mem_component_free(p4, MemType.CUDA) == Status.OK
    assert mc.xccl_mem_component_free(p2, MemType.CUDA) == Status.OK
    assert _calls(lib)[2] == n0[2] + 2


def test_host_alloc_and_missing_component(fake):
    st, p = mc.xccl_mem_component_alloc(64, MemType.HOST)
    assert st == Status.OK and p
    ctypes.memset(p, 0xAB, 64)
    assert mc.xccl_mem_component_free(p, MemType.HOST) == Status.OK
    st, _ = mc.xccl_mem_component_alloc(64, MemType.ROCM_MANAGED)
    assert st == Status.ERR_UNSUPPORTED          # mem_component.c:64-66
    assert mc.xccl_mem_component_free(1, MemType.ROCM_MANAGED) == Status.ERR_UNSUPPORTED


def test_mem_type_probe_order(fake):
    """mem_component.c:150-174: first component in enum order that recognises
    the pointer wins; nobody -> HOST."""
    lib_cuda, lib_mgd = fake[MemType.CUDA], fake[MemType.CUDA_MANAGED]
    lib_cuda.fake_arena_ptr.restype = ctypes.c_void_p
    lib_mgd.fake_arena_ptr.restype = ctypes.c_void_p
    st, mt = mc.xccl_mem_component_type(lib_cuda.fake_arena_ptr() + 8)
    assert (st, mt) == (Status.OK, MemType.CUDA)
    st, mt = mc.xccl_mem_component_type(lib_mgd.fake_arena_ptr() + 8)
    assert (st, mt) == (Status.OK, MemType.CUDA_MANAGED)
    buf = ctypes.create_string_buffer(16)
    st, mt = mc.xccl_mem_component_type(ctypes.addressof(buf))
    assert (st, mt) == (Status.OK, MemType.HOST)


def test_reduce_forwarding_and_error_codes(fake):
    lib = fake[MemType.CUDA]
    n0 = _calls(lib)
    assert mc.xccl_mem_component_reduce(0x1000, 0x2000, 0x3000, 77, Dt.INT32, Op.SUM, MemType.CUDA) == Status.OK
    args = list((ctypes.c_size_t * 8).in_dll(lib, "fake_last_args"))
    assert args[:6] == [0x1000, 0x2000, 0x3000, 77, int(Dt.INT32), int(Op.SUM)]
    assert mc.xccl_mem_component_reduce_multi(0x1000, 0x2000, 0x3000, 3, 55, 220, Dt.FLOAT32, Op.MAX,
                                              MemType.CUDA) == Status.OK
    args = list((ctypes.c_size_t * 8).in_dll(lib, "fake_last_args"))
    assert args == [0x1000, 0x2000, 0x3000, 3, 55, 220, int(Dt.FLOAT32), int(Op.MAX)]
    n1 = _calls(lib)
    assert (n1[4], n1[5]) == (n0[4] + 1, n0[5] + 1)
    # size == 0: OK before any lookup, even for a memory type with no component (mem_component.c:129-131)
    assert mc.xccl_mem_component_reduce_multi(0, 0, 0, 3, 0, 0, Dt.FLOAT32, Op.SUM, MemType.ROCM_MANAGED) == Status.OK
    assert _calls(lib)[5] == n1[5]
    # no component for the memory type
    assert mc.xccl_mem_component_reduce(1, 2, 3, 4, Dt.INT32, Op.SUM, MemType.ROCM_MANAGED) == Status.ERR_UNSUPPORTED
    assert mc.xccl_mem_component_reduce_multi(1, 2, 3, 1, 4, 16, Dt.INT32, Op.SUM,
                                              MemType.ROCM_MANAGED) == Status.ERR_UNSUPPORTED
    # host memory: this dispatcher carries no CPU arithmetic
    assert mc.xccl_mem_component_reduce(1, 2, 3, 4, Dt.INT32, Op.SUM, MemType.HOST) == Status.ERR_UNSUPPORTED
    assert mc.xccl_mem_component_reduce_multi(1, 2, 3, 1, 4, 16, Dt.INT32, Op.SUM,
                                              MemType.HOST) == Status.ERR_UNSUPPORTED


def test_stream_ordered_entries_and_their_fallback_rule(fake):
    """The *_nb dispatcher entries (the ones integration/xccl-rocm.patch adds to
    reference src/utils/mem_component.c): one fallback rule, followed here by
    every branch."""
    plain, ext = fake[MemType.CUDA], fake[MemType.CUDA_MANAGED]
    s = mc.Stream(0x1234, StreamType.CUDA)
    # a component without the extension, no stream named: the blocking entry runs, no event
    n0 = _calls(plain)
    st, ev = mc.xccl_mem_component_reduce_multi_nb(0x10, 0x20, 0x30, 3, 55, 220, Dt.FLOAT32, Op.MAX, MemType.CUDA)
    assert (st, ev) == (Status.OK, None) and _calls(plain)[5] == n0[5] + 1
    assert list((ctypes.c_size_t * 8).in_dll(plain, "fake_last_args")) == [0x10, 0x20, 0x30, 3, 55, 220,
                                                                           int(Dt.FLOAT32), int(Op.MAX)]
    st, ev = mc.xccl_mem_component_reduce_nb(0x10, 0x20, 0x30, 77, Dt.INT32, Op.SUM, MemType.CUDA)
    assert (st, ev) == (Status.OK, None) and _calls(plain)[4] == n0[4] + 1
    # ... a stream named: nothing can keep that order
    st, ev = mc.xccl_mem_component_reduce_multi_nb(0x10, 0x20, 0x30, 3, 55, 220, Dt.FLOAT32, Op.MAX, MemType.CUDA, s)
    assert (st, ev) == (Status.ERR_NOT_IMPLEMENTED, None) and _calls(plain)[5] == n0[5] + 1
    # no component / host memory: what the blocking dispatcher entry says
    st, ev = mc.xccl_mem_component_reduce_nb(1, 2, 3, 4, Dt.INT32, Op.SUM, MemType.ROCM_MANAGED)
    assert (st, ev) == (Status.ERR_UNSUPPORTED, None)
    st, ev = mc.xccl_mem_component_reduce_multi_nb(1, 2, 3, 1, 4, 16, Dt.INT32, Op.SUM, MemType.HOST)
    assert (st, ev) == (Status.ERR_UNSUPPORTED, None)
    # a component with the extension: forwarded with the stream, event stamped with the memory type
    ext.fake_set_nb_status(int(Status.OK))
    n0 = _calls(ext)
    st, ev = mc.xccl_mem_component_reduce_multi_nb(0x10, 0x20, 0x30, 3, 55, 220, Dt.FLOAT32, Op.MAX,
                                                   MemType.CUDA_MANAGED)
    assert st == Status.OK and ctypes.c_int.from_address(ev).value == MemType.CUDA_MANAGED
    assert _calls(ext)[14] == n0[14] + 1 and _calls(ext)[5] == n0[5]
    assert ctypes.c_void_p.in_dll(ext, "fake_last_stream").value is None
    st, ev = mc.xccl_mem_component_reduce_nb(0x10, 0x20, 0x30, 77, Dt.INT32, Op.SUM, MemType.CUDA_MANAGED, s)
    assert st == Status.OK and ev and _calls(ext)[13] == n0[13] + 1
    assert ctypes.c_void_p.in_dll(ext, "fake_last_stream").value == ctypes.addressof(s.xccl)
    st, ev = mc.xccl_mem_component_reduce_nb(0x10, 0x20, 0x30, 77, Dt.INT32, Op.SUM, MemType.CUDA_MANAGED, s,
                                             want_event=False)
    assert (st, ev) == (Status.OK, None) and _calls(ext)[13] == n0[13] + 2
    # an empty reduction: complete on return, nothing forwarded
    st, ev = mc.xccl_mem_component_reduce_multi_nb(0x10, 0x20, 0x30, 3, 0, 220, Dt.FLOAT32, Op.MAX,
                                                   MemType.CUDA_MANAGED)
    assert (st, ev) == (Status.OK, None) and _calls(ext)[14] == n0[14] + 1
    st, ev = mc.xccl_mem_component_reduce_nb(0x10, 0x20, 0x30, 0, Dt.INT32, Op.SUM, MemType.CUDA_MANAGED)
    assert (st, ev) == (Status.OK, None) and _calls(ext)[13] == n0[13] + 2
    # the component has no event left: without a stream the blocking entry runs instead ...
    ext.fake_set_nb_status(int(Status.ERR_NO_RESOURCE))
    n1 = _calls(ext)
    st, ev = mc.xccl_mem_component_reduce_multi_nb(0x10, 0x20, 0x30, 3, 55, 220, Dt.FLOAT32, Op.MAX,
                                                   MemType.CUDA_MANAGED)
    assert (st, ev) == (Status.OK, None) and _calls(ext)[14] == n1[14] + 1 and _calls(ext)[5] == n1[5] + 1
    st, ev = mc.xccl_mem_component_reduce_nb(0x10, 0x20, 0x30, 77, Dt.INT32, Op.SUM, MemType.CUDA_MANAGED)
    assert (st, ev) == (Status.OK, None) and _calls(ext)[13] == n1[13] + 1 and _calls(ext)[4] == n1[4] + 1
    # ... with one the caller is told
    st, ev = mc.xccl_mem_component_reduce_multi_nb(0x10, 0x20, 0x30, 3, 55, 220, Dt.FLOAT32, Op.MAX,
                                                   MemType.CUDA_MANAGED, s)
    assert (st, ev) == (Status.ERR_NO_RESOURCE, None) and _calls(ext)[5] == n1[5] + 1
    # any other failure is passed on
    ext.fake_set_nb_status(int(Status.ERR_UNSUPPORTED))
    st, ev = mc.xccl_mem_component_reduce_nb(0x10, 0x20, 0x30, 77, Dt.INT32, Op.SUM, MemType.CUDA_MANAGED)
    assert (st, ev) == (Status.ERR_UNSUPPORTED, None) and _calls(ext)[4] == n1[4] + 1
    ext.fake_set_nb_status(int(Status.OK))


def test_stream_routed_entries(fake):
    """mem_component.c:176-257: the stream's type picks the component; the
    dispatcher stamps mem_type into the returned event / request."""
    lib = fake[MemType.CUDA]
    s = mc.Stream(0x1234, StreamType.CUDA)
    st, ev = mc.xccl_mc_event_record(s)
    assert st == Status.OK and ctypes.c_int.from_address(ev).value == MemType.CUDA
    assert mc.xccl_mc_event_query(ev) == Status.INPROGRESS
    assert mc.xccl_mc_event_free(ev) == Status.OK
    assert mc.xccl_mc_event_wait(ev) == Status.ERR_NOT_IMPLEMENTED
    st, req = mc.xccl_mem_component_start_acitivity(s)
    assert st == Status.OK and ctypes.c_int.from_address(req).value == MemType.CUDA
    assert mc.xccl_mem_component_finish_acitivity(req) == Status.OK
    src = ctypes.create_string_buffer(b"0123456789abcdef")
    dst = ctypes.create_string_buffer(16)
    assert mc.xccl_mem_component_memcpy_async(ctypes.addressof(src), ctypes.addressof(dst), 16, s) == Status.OK
    assert dst.raw == src.raw[:16]
    n = _calls(lib)
    assert mc.xccl_mem_component_memcpy_async(ctypes.addressof(src), ctypes.addressof(dst), 0, s) == Status.OK
    assert _calls(lib)[6] == n[6]               # size 0 never reaches the component (:185-187)
    assert n[7] >= 1 and n[8] >= 1 and n[9] >= 1 and n[10] >= 1 and n[11] >= 1


def test_init_rejects_null_and_missing_dir():
    assert mc.dispatch_lib().xccl_mem_component_init(None) == Status.ERR_INVALID_PARAM
    assert mc.xccl_mem_component_init("/nonexistent/dir") == Status.OK   # nothing found is not an error


def test_libs_are_in_tree():
    for n in ("xccl_rocm_mem_component.so", "libxccl_mc.so", "libxccl_rocm_benchkit.so"):
        assert os.path.isfile(os.path.join(LIB_DIR, n))


def test_cached_buffer_is_never_lent_twice(fake, tmp_path):
    """Collectives may be posted from several threads (the ucx team library
    advertises XCCL_THREAD_MODE_MULTIPLE, xccl_ucx_lib.c:631-632): 8 threads
    borrow and return small buffers through the dispatcher; nobody may ever
    find another thread's bytes in the buffer it holds."""
    out = str(tmp_path / "libdispatch_stress.so")
    subprocess.run(["gcc", "-shared", "-fPIC", "-O2", "-Wall", "-Wextra", "-Werror", "-I", INC, "-o", out,
                    os.path.join(ROOT, "tests", "dispatch_stress.c"), "-L", LIB_DIR, "-lxccl_mc", "-lpthread",
                    "-Wl,-rpath," + LIB_DIR], check=True)
    mc.dispatch_lib()                                   # the copy of libxccl_mc.so the fixture initialised
    lib = ctypes.CDLL(out)
    lib.dispatch_stress.restype = ctypes.c_long
    loans = ctypes.c_long(0)
    errors = lib.dispatch_stress(8, 200000, int(MemType.CUDA), ctypes.byref(loans))
    assert errors == 0
    assert loans.value > 0                              # the cached buffer did go round
    vt = mc.dispatch_lib().xccl_mem_component_get(int(MemType.CUDA)).contents
    assert vt.cache.used == 0
