"""The UCX team library's reduction call sites, replayed over loopback ranks on
one GPU (libxccl_ucx_replay.so), in the shape of the reference's device tests:
test/test_mpi_cuda_allreduce.c (INT32 SUM, count 32, rank r contributes
r + 1 + 12345 + i, compare with the MPI result) and test/test_mpi_cuda_reduce.c
(the same for every root)."""
import numpy as np
import pytest

from gpu_util import NP
from xccl_amd import hip
from xccl_amd.types import Dt, Op, Status, dt_size, supported_pairs, FP_DTYPES

pytestmark = pytest.mark.gpu

ALLREDUCE = ("allreduce_knomial", "allreduce_sra")
REDUCE = ("reduce_knomial", "reduce_linear")


class Ranks:
    """P ranks, each with a source and a destination vector in device memory."""

    def __init__(self, host_src: np.ndarray, in_place=False, canary=0xA5):
        self.P, self.count = host_src.shape
        self.nbytes = host_src[0].nbytes
        self.src = [hip.DeviceBuffer(self.nbytes) for _ in range(self.P)]
        self.dst = self.src if in_place else [hip.DeviceBuffer(self.nbytes) for _ in range(self.P)]
        for r in range(self.P):
            self.src[r].upload(host_src[r])
            if not in_place:
                hip.memset(self.dst[r].ptr, canary, self.nbytes)
        self.dtype = host_src.dtype

    def src_ptrs(self):
        return [b.ptr for b in self.src]

    def dst_ptrs(self):
        return [b.ptr for b in self.dst]

    def result(self, r):
        return self.dst[r].download(self.dtype, self.count)

    def source(self, r):
        return self.src[r].download(self.dtype, self.count)

    def close(self):
        for b in set(self.src) | set(self.dst):
            b.close()


def _kat(P, count=32):
    return np.array([[r + 1 + 12345 + i for i in range(count)] for r in range(P)], dtype=np.int32)


@pytest.mark.parametrize("alg", ALLREDUCE)
@pytest.mark.parametrize("stream_ordered", [False, True], ids=["blocking", "stream_ordered"])
def test_allreduce_known_answer_every_team_size(rocm, alg, stream_ordered):
    """test_mpi_cuda_allreduce.c:35-76 / test_mt.c:58 for team sizes 2..17 and
    radices 2..8: every rank must end with P(P+1)/2 + P(i + 12345)."""
    for P in range(2, 18):
        expect = [P * (P + 1) // 2 + P * (i + 12345) for i in range(32)]
        for radix in (2, 3, 4, 5, 8):
            rk = Ranks(_kat(P))
            st, stats = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), 32, Dt.INT32, Op.SUM, radix=radix,
                                        stream_ordered=stream_ordered)
            assert st == Status.OK, (alg, P, radix, st)
            for r in range(P):
                assert rk.result(r).tolist() == expect, (alg, P, radix, r)
                assert rk.source(r).tolist() == _kat(P)[r].tolist(), "source buffer modified"
            assert stats["reduce_multi_calls"] > 0 and stats["messages"] > 0
            rk.close()


@pytest.mark.parametrize("alg", REDUCE)
@pytest.mark.parametrize("stream_ordered", [False, True], ids=["blocking", "stream_ordered"])
def test_reduce_known_answer_every_root(rocm, alg, stream_ordered):
    """test_mpi_cuda_reduce.c:47-78: all roots; only the root's destination is
    written, the others keep their canary."""
    for P in (2, 3, 4, 5, 7, 8, 9, 16, 17):
        expect = [P * (P + 1) // 2 + P * (i + 12345) for i in range(32)]
        for radix in (2, 4, 5):
            for root in range(P):
                rk = Ranks(_kat(P))
                st, stats = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), 32, Dt.INT32, Op.SUM, radix=radix,
                                            root=root, stream_ordered=stream_ordered)
                assert st == Status.OK, (alg, P, radix, root, st)
                assert rk.result(root).tolist() == expect, (alg, P, radix, root)
                for r in range(P):
                    if r != root:
                        assert (rk.result(r).view(np.uint8) == 0xA5).all(), "non-root destination written"
                if alg == "reduce_linear":
                    assert stats["reduce_calls"] == P - 1 and stats["inplace_sbuf2"] == P - 1
                rk.close()


def _random_ranks(oracle, P, count, dt, seed):
    return np.stack([oracle.fill(count, dt, seed, r) for r in range(P)])


@pytest.mark.parametrize("alg", ALLREDUCE + REDUCE)
def test_order_independent_operators_and_ragged_sizes(rocm, oracle, alg):
    """Integer SUM (wrapping), BXOR, MAX, MIN and LOR give the same bits in any
    fold order, so numpy's reduction over the rank axis is the expected value
    whatever tree the algorithm builds.  Counts that do not divide by the radix
    exercise the uneven scatter-reduce segments."""
    cases = [(Dt.INT32, Op.SUM, np.add), (Dt.UINT8, Op.BXOR, np.bitwise_xor), (Dt.INT16, Op.MAX, np.maximum),
             (Dt.UINT64, Op.MIN, np.minimum), (Dt.INT64, Op.SUM, np.add), (Dt.FLOAT64, Op.MAX, np.maximum),
             (Dt.FLOAT16, Op.MIN, np.minimum)]
    for P, radix in ((3, 2), (4, 4), (6, 4), (7, 3), (8, 4), (9, 4), (13, 5), (16, 4), (17, 8)):
        for count in (1, 5, 33, 1000, 4099):
            dt, op, fn = cases[(P + count) % len(cases)]
            host = _random_ranks(oracle, P, count, dt, seed=P * 1000 + count)
            with np.errstate(over="ignore"):
                want = fn.reduce(host, axis=0, dtype=host.dtype)   # keep the element width: integer SUM wraps
            rk = Ranks(host)
            st, stats = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), count, dt, op, radix=radix, root=P // 2)
            assert st == Status.OK, (alg, P, radix, count, st)
            who = range(P) if alg in ALLREDUCE else [P // 2]
            for r in who:
                assert rk.result(r).tobytes() == want.tobytes(), (alg, P, radix, count, Dt(dt).name, Op(op).name, r)
            rk.close()


def _expected_any_order(host, dt, op):
    """The reduction over the rank axis for an operator whose bits do not
    depend on the fold order, computed by numpy alone; for floating-point SUM
    and PROD (order-dependent) a float64 value and an error bound instead."""
    P = host.shape[0]
    if int(dt) in [int(d) for d in FP_DTYPES] and op in (Op.SUM, Op.PROD):
        x = host.astype(np.float64)
        u = {2: 2.0 ** -11, 4: 2.0 ** -24, 8: 2.0 ** -53}[host.itemsize]
        tiny = float(np.finfo(host.dtype).smallest_subnormal)
        # binary64 inputs: the float64 value below carries P-1 roundings of its own, hence twice the bound
        k = (2 if host.itemsize == 8 else 1) * (P - 1)
        if op == Op.SUM:
            return x.sum(axis=0), k * u * np.abs(x).sum(axis=0) + k * tiny
        # every multiplication is off by at most u relative (to first order), or half a subnormal step absolute
        return x.prod(axis=0), 1.01 * k * u * np.abs(x.prod(axis=0)) + k * tiny
    with np.errstate(over="ignore"):
        if op == Op.SUM:
            return np.add.reduce(host, axis=0, dtype=host.dtype), None
        if op == Op.PROD:
            return np.multiply.reduce(host, axis=0, dtype=host.dtype), None
    if op == Op.MAX:
        return np.maximum.reduce(host, axis=0), None
    if op == Op.MIN:
        return np.minimum.reduce(host, axis=0), None
    if op == Op.BAND:
        return np.bitwise_and.reduce(host, axis=0), None
    if op == Op.BOR:
        return np.bitwise_or.reduce(host, axis=0), None
    if op == Op.BXOR:
        return np.bitwise_xor.reduce(host, axis=0), None
    truth = host != 0
    if op == Op.LAND:
        return truth.all(axis=0).astype(host.dtype), None
    if op == Op.LOR:
        return truth.any(axis=0).astype(host.dtype), None
    assert op == Op.LXOR
    return (truth.sum(axis=0) % 2).astype(host.dtype), None


@pytest.mark.parametrize("stream_ordered", [False, True], ids=["blocking", "stream_ordered"])
@pytest.mark.parametrize("alg", ALLREDUCE + REDUCE)
def test_every_dtype_op_through_every_call_site(rocm, oracle, alg, stream_ordered):
    """test_mpi_cuda_allreduce.c:45-76 / test_mpi_cuda_reduce.c:47-78 "for every
    (dtype, op)": all 92 supported pairs through each algorithm's call sites
    (their in-place aliasing and scratch strides included), 5 ranks at radix 4
    (one extra rank handing its vector to a proxy) and 8 ranks at radix 4, a
    count that leaves ragged segments.  Integer operators, and floating-point
    MAX/MIN, must match numpy's reduction bit for bit whatever tree the
    algorithm builds; floating-point SUM/PROD must lie within the error bound
    of P-1 roundings."""
    count = 257
    for P in (5, 8):
        root = P - 2
        for dt, op in supported_pairs():
            sparse = op in (Op.LAND, Op.LOR, Op.LXOR)
            host = np.stack([oracle.fill(count, dt, 900 + P, r, sparse) for r in range(P)])
            want, bound = _expected_any_order(host, dt, op)
            rk = Ranks(host)
            st, _ = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), count, dt, op, radix=4, root=root,
                                    stream_ordered=stream_ordered)
            assert st == Status.OK, (alg, P, Dt(dt).name, Op(op).name, st)
            for r in (range(P) if alg in ALLREDUCE else [root]):
                got = rk.result(r)
                if bound is None:
                    assert got.tobytes() == want.tobytes(), (alg, P, Dt(dt).name, Op(op).name, r)
                else:
                    assert (np.abs(got.astype(np.float64) - want) <= bound).all(), (alg, P, Dt(dt).name, Op(op).name, r)
            rk.close()


@pytest.mark.parametrize("alg", ALLREDUCE)
def test_in_place_allreduce(rocm, oracle, alg):
    """src == dst on every rank: the scatter-reduce must move its work space
    out of dst (allreduce_sra.c:178-186); the k-nomial rounds then alias rbuf
    with sbuf1 from the first round on."""
    for P, radix, count in ((4, 4, 1000), (6, 4, 4099), (8, 2, 257), (9, 4, 100000)):
        host = _random_ranks(oracle, P, count, Dt.INT32, seed=77 + P)
        want = np.add.reduce(host, axis=0, dtype=host.dtype)
        rk = Ranks(host, in_place=True)
        st, stats = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), count, Dt.INT32, Op.SUM, radix=radix)
        assert st == Status.OK
        for r in range(P):
            assert np.array_equal(rk.result(r), want), (alg, P, radix, count, r)
        assert stats["inplace_sbuf1"] + stats["inplace_sbuf2"] > 0
        rk.close()


@pytest.mark.parametrize("alg", ALLREDUCE + REDUCE)
def test_float_sum_within_bound_and_exact_on_integers(rocm, oracle, alg):
    """fp32 SUM: the fold order depends on the algorithm (as it does across
    ranks in the reference), so random values are checked against a float64
    sum with |err| <= (P-1) * 2^-24 * sum|x_i|; small integers are exact in
    every order."""
    P, radix, count = 8, 4, 50000
    host = _random_ranks(oracle, P, count, Dt.FLOAT32, seed=5)
    exact = host.astype(np.float64).sum(axis=0)
    bound = (P - 1) * 2.0 ** -24 * np.abs(host.astype(np.float64)).sum(axis=0)
    rk = Ranks(host)
    st, _ = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), count, Dt.FLOAT32, Op.SUM, radix=radix, root=3)
    assert st == Status.OK
    for r in (range(P) if alg in ALLREDUCE else [3]):
        assert (np.abs(rk.result(r).astype(np.float64) - exact) <= bound).all()
    rk.close()
    ints = (_random_ranks(oracle, P, count, Dt.INT8, seed=6).astype(np.float32))
    rk = Ranks(ints)
    st, _ = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), count, Dt.FLOAT32, Op.SUM, radix=radix, root=3)
    assert st == Status.OK
    for r in (range(P) if alg in ALLREDUCE else [3]):
        assert np.array_equal(rk.result(r), ints.sum(axis=0, dtype=np.float32))
    rk.close()


def test_call_shapes_of_a_radix4_team_of_8(rocm):
    """What the state machines ask of the component, counted: 8 ranks, radix 4
    -> two k-nomial rounds; round one folds 3 received vectors into the own
    one, round two folds 1 (allreduce_knomial.c:129-135: n = active_reqs/2)."""
    P, count = 8, 4096
    rk = Ranks(np.ones((P, count), dtype=np.int32))
    st, stats = rocm.replay_run("allreduce_knomial", rk.src_ptrs(), rk.dst_ptrs(), count, Dt.INT32, Op.SUM, radix=4)
    assert st == Status.OK
    assert stats["reduce_multi_calls"] == 16 and stats["reduce_calls"] == 0 and stats["max_multi_vectors"] == 3
    assert stats["inplace_sbuf1"] == 8            # second round: rbuf == sbuf1 == dst
    assert stats["messages"] == 8 * 3 + 8 * 1 and stats["scratch_allocs"] == 8
    assert (rk.result(5) == P).all()
    rk.close()
    # scatter-reduce: round one leaves the result at the start of the work space, which is where the
    # first arrival sits (rbuf == sbuf2); message bytes shrink by the radix per round
    rk = Ranks(np.ones((P, count), dtype=np.int32))
    st, stats = rocm.replay_run("allreduce_sra", rk.src_ptrs(), rk.dst_ptrs(), count, Dt.INT32, Op.SUM, radix=4)
    assert st == Status.OK and stats["reduce_multi_calls"] == 16 and stats["inplace_sbuf2"] >= 8
    assert stats["scratch_allocs"] == 0           # dst doubles as work space when src != dst
    assert (rk.result(2) == P).all()
    rk.close()
    # 6 ranks: 2 extras hand their vectors to proxies, who fold them in with a 2-source reduce first
    rk = Ranks(np.ones((6, count), dtype=np.int32))
    st, stats = rocm.replay_run("allreduce_knomial", rk.src_ptrs(), rk.dst_ptrs(), count, Dt.INT32, Op.SUM, radix=4)
    assert st == Status.OK and stats["reduce_calls"] == 2 and stats["reduce_multi_calls"] == 4
    assert all((rk.result(r) == 6).all() for r in range(6))
    rk.close()


def test_large_vectors_stream_ordered_overlap(rocm, oracle):
    """64 MiB per rank, 4 ranks: the reductions take long enough that ranks
    return with theirs still in flight, and other ranks' progress functions
    run meanwhile -- the point of the stream-ordered call sites."""
    P, count = 4, 16 * 1024 * 1024
    host = _random_ranks(oracle, P, count, Dt.INT32, seed=9)
    want = np.add.reduce(host, axis=0, dtype=host.dtype)
    for alg in ALLREDUCE:
        rk = Ranks(host)
        st, stats = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), count, Dt.INT32, Op.SUM, radix=4)
        assert st == Status.OK
        for r in range(P):
            assert np.array_equal(rk.result(r), want)
        assert stats["reduce_inflight_returns"] > 0
        rk.close()


def test_four_threads_run_collectives_at_once(rocm):
    """test/test_mt.c: 4 threads, each with a team of its own, run allreduce
    after allreduce (INT32 SUM, count 32, the closed form of test_mt.c:58) --
    here each thread drives its own set of loopback ranks through the one
    component.  Together they want more pooled events than the component has,
    so transport marks fall back to stream waits and reductions to the
    blocking entry now and then; every result must still be right."""
    import threading
    P, iters = 6, 12
    expect = [P * (P + 1) // 2 + P * (i + 12345) for i in range(32)]
    teams = [Ranks(_kat(P)) for _ in range(4)]
    errors = []

    def worker(t):
        rk = teams[t]
        try:
            for it in range(iters):
                alg = ALLREDUCE[(t + it) % 2]
                st, _ = rocm.replay_run(alg, rk.src_ptrs(), rk.dst_ptrs(), 32, Dt.INT32, Op.SUM, radix=2 + (t + it) % 3,
                                        stream_ordered=bool((t + it // 2) % 2))
                if st != Status.OK:
                    errors.append((t, it, alg, "status", st))
                    return
                for r in range(P):
                    if rk.result(r).tolist() != expect:
                        errors.append((t, it, alg, "rank", r))
                        return
        except Exception as e:      # noqa: BLE001 -- reported by the main thread
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(100)
    assert not any(th.is_alive() for th in threads), "a thread is stuck"
    assert errors == []
    for rk in teams:
        rk.close()


def test_c_program_in_the_shape_of_the_reference_tests():
    """tests/c/test_rocm_allreduce.c: a C program laid out like
    test/test_mpi_cuda_allreduce.c and test/test_mpi_cuda_reduce.c, driving the
    dispatcher and the component from C only (built by xccl_amd/csrc/Makefile)."""
    import os
    import subprocess
    from xccl_amd.build import LIB_DIR
    exe = os.path.join(LIB_DIR, "test_rocm_allreduce")
    for team, count in ((8, 32), (6, 32), (17, 32), (5, 100000)):
        out = subprocess.run([exe, LIB_DIR, str(team), str(count)], capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stdout + out.stderr
        assert "Correctness check: PASSED" in out.stdout
    # "... then every (dtype, op)": 8 integer types x 10 operators + FLOAT32/FLOAT64 x MAX, MIN, SUM = 86 cases,
    # each through the four algorithms in both reduction modes
    for team, count in ((8, 32), (5, 1001)):
        out = subprocess.run([exe, LIB_DIR, str(team), str(count), "ALL", "ALL"], capture_output=True, text=True,
                             timeout=300)
        assert out.returncode == 0, out.stdout + out.stderr
        assert "Correctness check: PASSED" in out.stdout and "86 dtype/op cases" in out.stdout
    out = subprocess.run([exe, LIB_DIR, "4", "64", "UINT16", "LXOR"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "1 dtype/op case)" in out.stdout, out.stdout + out.stderr
