"""Pure-Python model of the reference's operators on Python ints, written from
the C language rules (integer promotion, two's-complement truncation on
assignment), independent of the oracle's C code.  reference
src/utils/reduce.h:14-23 gives the operator macros; the first macro argument
is `a`."""

INT_INFO = {  # xccl_dt_t -> (bits, signed)
    0: (8, True), 1: (16, True), 2: (32, True), 3: (64, True),
    5: (8, False), 6: (16, False), 7: (32, False), 8: (64, False),
}

OP_MAX, OP_MIN, OP_SUM, OP_PROD = 0, 1, 2, 3
OP_LAND, OP_LOR, OP_LXOR, OP_BAND, OP_BOR, OP_BXOR = 7, 8, 9, 10, 11, 12
INT_OPS = (OP_MAX, OP_MIN, OP_SUM, OP_PROD, OP_LAND, OP_LOR, OP_LXOR, OP_BAND, OP_BOR, OP_BXOR)
FP_OPS = (OP_MAX, OP_MIN, OP_SUM, OP_PROD)


def wrap(v: int, bits: int, signed: bool) -> int:
    """Value of (T)v for a `bits`-wide two's-complement / unsigned T."""
    v &= (1 << bits) - 1
    if signed and v >> (bits - 1):
        v -= 1 << bits
    return v


def int_op(op: int, a: int, b: int, bits: int, signed: bool) -> int:
    if op == OP_MAX:
        r = a if a > b else b
    elif op == OP_MIN:
        r = a if a < b else b
    elif op == OP_SUM:
        r = a + b
    elif op == OP_PROD:
        r = a * b
    elif op == OP_LAND:
        r = 1 if (a != 0 and b != 0) else 0
    elif op == OP_LOR:
        r = 1 if (a != 0 or b != 0) else 0
    elif op == OP_LXOR:
        r = 1 if ((a == 0) != (b == 0)) else 0
    elif op == OP_BAND:
        r = a & b
    elif op == OP_BOR:
        r = a | b
    elif op == OP_BXOR:
        r = a ^ b
    else:
        raise ValueError(op)
    return wrap(r, bits, signed)


def fold(op_fn, s1, s2_list):
    """reference src/utils/mem_component.c:133-139: acc = OP(s1, s2[0]); then
    acc = OP(s2[j], acc) -- new source first."""
    acc = op_fn(s1, s2_list[0])
    for x in s2_list[1:]:
        acc = op_fn(x, acc)
    return acc


def edge_values(bits: int, signed: bool):
    if signed:
        lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
        return [lo, lo + 1, -2, -1, 0, 1, 2, hi - 1, hi, 0x55 & hi, -0x56 if bits == 8 else -(0x5555 & hi)]
    hi = (1 << bits) - 1
    return [0, 1, 2, 3, hi >> 1, (hi >> 1) + 1, hi - 1, hi, 0x55 & hi, 0xAA & hi]
