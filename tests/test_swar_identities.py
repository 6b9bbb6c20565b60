"""The whole-register forms the kernels use for 8- and 16-bit logical
operators and the 8-bit SUM (xccl_amd/csrc/reduce_kernel.hpp: nz8, nz16,
vfold<uint8_t, OpSum>) rest on bit identities; here each identity is checked
against the element-wise definition of reference src/utils/reduce.h:14-23,
exhaustively for bytes and on edge + random values for 16-bit elements.  (The
device code itself is checked on the GPU by the parity tests.)"""
import numpy as np


def _pack(elems, dtype):
    return np.ascontiguousarray(elems, dtype=dtype).view(np.uint32)


def _nz(x, low, shift, one):
    return ((((x & low) + low) | x) >> shift) & one


def _cases8():
    a, b = np.meshgrid(np.arange(256, dtype=np.uint8), np.arange(256, dtype=np.uint8))
    return a.ravel(), b.ravel()          # 65,536 pairs = 16,384 registers of four bytes


def _cases16():
    rng = np.random.default_rng(7)
    edge = np.array([0, 1, 2, 0x7f, 0x80, 0xff, 0x100, 0x7fff, 0x8000, 0x8001, 0xfffe, 0xffff], dtype=np.uint16)
    a, b = np.meshgrid(edge, edge)
    ra = rng.integers(0, 1 << 16, 100000, dtype=np.uint16)
    rb = rng.integers(0, 1 << 16, 100000, dtype=np.uint16)
    rb[::3] = 0
    ra[::5] = 0
    return np.concatenate([a.ravel(), ra]), np.concatenate([b.ravel(), rb])


def test_nonzero_mask_and_logical_operators_bytes():
    a, b = _cases8()
    A, B = _pack(a, np.uint8), _pack(b, np.uint8)
    nz = lambda x: _nz(x, np.uint32(0x7f7f7f7f), np.uint32(7), np.uint32(0x01010101))   # noqa: E731
    assert np.array_equal(nz(A).view(np.uint8), (a != 0).astype(np.uint8))
    assert np.array_equal((nz(A) & nz(B)).view(np.uint8), ((a != 0) & (b != 0)).astype(np.uint8))       # LAND
    assert np.array_equal(nz(A | B).view(np.uint8), ((a != 0) | (b != 0)).astype(np.uint8))             # LOR
    assert np.array_equal((nz(A) ^ nz(B)).view(np.uint8), ((a == 0) != (b == 0)).astype(np.uint8))      # LXOR


def test_nonzero_mask_and_logical_operators_16bit():
    a, b = _cases16()
    A, B = _pack(a, np.uint16), _pack(b, np.uint16)
    nz = lambda x: _nz(x, np.uint32(0x7fff7fff), np.uint32(15), np.uint32(0x00010001))  # noqa: E731
    assert np.array_equal(nz(A).view(np.uint16), (a != 0).astype(np.uint16))
    assert np.array_equal((nz(A) & nz(B)).view(np.uint16), ((a != 0) & (b != 0)).astype(np.uint16))
    assert np.array_equal(nz(A | B).view(np.uint16), ((a != 0) | (b != 0)).astype(np.uint16))
    assert np.array_equal((nz(A) ^ nz(B)).view(np.uint16), ((a == 0) != (b == 0)).astype(np.uint16))


def test_bytewise_wrapping_sum():
    a, b = _cases8()
    A, B = _pack(a, np.uint8), _pack(b, np.uint8)
    low, top = np.uint32(0x7f7f7f7f), np.uint32(0x80808080)
    got = ((A & low) + (B & low)) ^ ((A ^ B) & top)
    assert np.array_equal(got.view(np.uint8), a + b)        # uint8 addition wraps, as (T)(a + b) does
    # no carry may cross a byte: a register of 0xff bytes plus a register of 0x01 bytes is all zero
    one = np.array([0x01010101], dtype=np.uint32)
    ff = np.array([0xffffffff], dtype=np.uint32)
    assert (((ff & low) + (one & low)) ^ ((ff ^ one) & top))[0] == 0
