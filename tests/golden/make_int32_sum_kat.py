#!/usr/bin/env python3
"""Writes tests/golden/int32_sum_count32.json: the one known-answer case the
reference's own tests hold for the reduction path.

Inputs and expected outputs are those of reference test/test_mpi_allreduce.c:18-21,
test/test_mpi_cuda_allreduce.c:35-39 (every rank r of P contributes
sbuf[i] = r + 1 + 12345 + i, count 32, XCCL_DT_INT32, XCCL_OP_SUM) and of the
closed form those tests check the result against, test/test_mt.c:58
(size*(size+1)/2 + size*(j+12345)).  Team sizes 2..17: 17 is the largest team
the default request limit of the UCX team library allows at full radix
(src/team_lib/ucx/xccl_ucx_lib.h:65).  Pure arithmetic; needs nothing but Python.
"""
import json
import os

COUNT = 32


def main():
    cases = []
    for p in range(2, 18):
        inputs = [[r + 1 + 12345 + i for i in range(COUNT)] for r in range(p)]
        closed = [p * (p + 1) // 2 + p * (j + 12345) for j in range(COUNT)]
        assert closed == [sum(col) for col in zip(*inputs)]      # the tests' closed form IS the plain sum
        cases.append({
            "team_size": p, "count": COUNT, "dtype": "INT32", "op": "SUM",
            "inputs": inputs,
            "expected": closed,
        })
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "int32_sum_count32.json")
    with open(out, "w") as f:
        json.dump({"source": "reference test/test_mt.c:58, test/test_mpi_cuda_allreduce.c:35-39", "cases": cases}, f)
    print("wrote", out, len(cases), "cases")


if __name__ == "__main__":
    main()
