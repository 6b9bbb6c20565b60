"""ctypes binding of oracle/liboracle.so (the CPU restatement of the reference's
``xccl_dt_reduce`` and host ``reduce_multi``).

TEST INFRASTRUCTURE, NOT PRODUCT.  Importers: tests/, __graft_entry__.smoke(),
bench.py's cpu_baseline leg.  Nothing under xccl_amd/ may import this.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SO = os.path.join(HERE, "liboracle.so")

_vp, _sz, _int, _u64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_uint64
_lib = None

# xccl_dt_t value -> numpy dtype holding its bits (binary16 as float16)
NP_DTYPE = {
    0: np.int8, 1: np.int16, 2: np.int32, 3: np.int64,
    5: np.uint8, 6: np.uint16, 7: np.uint32, 8: np.uint64,
    10: np.float16, 11: np.float32, 12: np.float64,
}


def build(force: bool = False) -> None:
    """Compiles liboracle.so with gcc (oracle/Makefile)."""
    cmd = ["make", "-C", HERE]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.isfile(SO):
            build()
        l = ctypes.CDLL(SO)
        l.oracle_dtype_in_reference.argtypes = [_int]
        l.oracle_dt_reduce.argtypes = [_vp, _vp, _vp, _sz, _int, _int]
        l.oracle_reduce_multi.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int]
        l.oracle_reduce_multi_mt.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _int]
        l.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        l.oracle_half_to_float.restype = ctypes.c_float
        l.oracle_float_to_half.argtypes = [ctypes.c_float]
        l.oracle_float_to_half.restype = ctypes.c_uint16
        l.oracle_fill.argtypes = [_vp, _sz, _int, _u64, _u64, _int, _int]
        l.oracle_splitmix64.argtypes = [_u64]
        l.oracle_splitmix64.restype = _u64
        _lib = l
    return _lib


def _ptr(a: np.ndarray, byte_offset: int = 0) -> int:
    return a.ctypes.data + byte_offset


def dt_reduce(sbuf1: np.ndarray, sbuf2: np.ndarray, target: np.ndarray, count: int, dtype: int, op: int) -> int:
    """xccl_dt_reduce on numpy buffers (any of which may be the same array)."""
    return lib().oracle_dt_reduce(_ptr(sbuf1), _ptr(sbuf2), _ptr(target), count, int(dtype), int(op))


def reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, *, off1=0, off2=0, offr=0, threads=1) -> int:
    """Host xccl_mem_component_reduce_multi.  sbuf1/sbuf2/rbuf are numpy arrays
    (may alias); off* are byte offsets into them; stride is in bytes."""
    f = lib().oracle_reduce_multi_mt
    return f(_ptr(sbuf1, off1), _ptr(sbuf2, off2), _ptr(rbuf, offr), count, size, stride, int(dtype), int(op),
             int(threads))


def reduce_multi_ptr(p1: int, p2: int, pr: int, count, size, stride, dtype, op, threads=1) -> int:
    return lib().oracle_reduce_multi_mt(p1, p2, pr, count, size, stride, int(dtype), int(op), int(threads))


def fill(count: int, dtype: int, seed: int, vec: int, sparse: bool = False, threads: int = 8,
         out: np.ndarray = None) -> np.ndarray:
    """Vector `vec` of synthetic stream `seed` (recipe in xccl_oracle.h)."""
    if out is None:
        out = np.empty(count, dtype=NP_DTYPE[int(dtype)])
    assert out.size >= count and out.dtype == NP_DTYPE[int(dtype)]
    rc = lib().oracle_fill(_ptr(out), count, int(dtype), seed, vec, int(bool(sparse)), threads)
    if rc != 0:
        raise ValueError("oracle_fill: unsupported dtype %d" % dtype)
    return out


def slab(nvec: int, count: int, dtype: int, seed: int, sparse: bool = False, threads: int = 8) -> np.ndarray:
    """nvec vectors back to back (stride = count*itemsize), vector v = fill(.., vec=v)."""
    a = np.empty((nvec, count), dtype=NP_DTYPE[int(dtype)])
    for v in range(nvec):
        fill(count, dtype, seed, v, sparse, threads, out=a[v])
    return a
