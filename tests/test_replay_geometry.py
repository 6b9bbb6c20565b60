"""Host-only checks of the k-nomial geometry and the scatter-reduce segment
arithmetic behind the call-site replay (no GPU): invariants the algorithms
need, worked examples, and -- where the reference tree is present -- the
structure of the reference's own macros evaluated in Python."""
import ctypes

import pytest

from xccl_amd import mc


def _geometry_model(radix, rank, size):
    """reference src/team_lib/ucx/allreduce/allreduce_knomial.h:10-34, evaluated step by step."""
    pk, fs = 1, radix
    while fs < size:
        pk += 1
        fs *= radix
    full_tree = fs // radix if fs != size else fs
    if fs != size and size // full_tree == 1:
        pk -= 1
    full = (size // full_tree) * full_tree
    role = 2 if rank >= full else (1 if (size > full and rank < size - full) else 0)
    return pk, full, role


def test_replay_symbols_exported():
    import os
    import re
    text = open(os.path.join(os.path.dirname(__file__), "..", "include", "xccl_rocm_ucx_replay.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = {n for n in re.findall(r"\b(xccl_replay_[a-z0-9_]+)\s*\(", text)}
    assert names == {"xccl_replay_run", "xccl_replay_knomial_geometry", "xccl_replay_sra_segment"}
    for n in names:
        assert hasattr(mc.replay_lib(), n)


def test_knomial_geometry_matches_macro_model_and_invariants():
    for radix in range(2, 9):
        for size in range(2, 70):
            r = min(radix, size)
            roles = []
            for rank in range(size):
                got = mc.knomial_geometry(r, rank, size)
                assert got == _geometry_model(r, rank, size), (r, rank, size)
                roles.append(got[2])
            rounds, full, _ = mc.knomial_geometry(r, 0, size)
            # ranks [0, full) exchange; every extra rank pairs with exactly one proxy
            assert full <= size <= 2 * full
            n_extra = roles.count(2)
            assert n_extra == size - full == roles.count(1)
            assert roles[:n_extra] == [1] * n_extra and roles[full:] == [2] * n_extra
            # after `rounds` rounds of groups of r, every base rank has heard from all of [0, full)
            reach = {rank: {rank} for rank in range(full)}
            pw = 1
            for _ in range(rounds):
                span = pw * r
                new = {}
                for rank in range(full):
                    acc = set(reach[rank])
                    for k in range(1, r):
                        peer = (rank + k * pw) % span + (rank - rank % span)
                        if peer < full:
                            acc |= reach[peer]
                    new[rank] = acc
                reach, pw = new, pw * r
            assert all(v == set(range(full)) for v in reach.values()), (r, size)


def test_worked_examples():
    # 8 ranks, radix 4: two complete subtrees of 4, two rounds, nobody extra
    assert [mc.knomial_geometry(4, r, 8) for r in (0, 7)] == [(2, 8, 0), (2, 8, 0)]
    # 6 ranks, radix 4: one subtree of 4, one round, ranks 4-5 extra, ranks 0-1 their proxies
    assert [mc.knomial_geometry(4, r, 6)[2] for r in range(6)] == [1, 1, 0, 0, 2, 2]
    assert mc.knomial_geometry(4, 0, 6)[:2] == (1, 4)
    # 16 ranks radix 4 -> 2 rounds; 17 ranks radix 4 -> 16 exchange, one extra
    assert mc.knomial_geometry(4, 0, 16)[:2] == (2, 16)
    assert mc.knomial_geometry(4, 16, 17) == (2, 16, 2)


@pytest.mark.parametrize("radix", [2, 3, 4, 5, 8])
def test_sra_segments_partition_the_vector(radix):
    """After the scatter-reduce every exchanging rank owns one segment; the
    segments must tile [0, count) without gap or overlap, whatever the
    remainders are -- otherwise the allgather cannot rebuild the vector."""
    for size in list(range(2, 20)) + [32, 33]:
        r = min(radix, size)
        _, full, _ = mc.knomial_geometry(r, 0, size)
        for count in (full, 32, 1000, 1023, 65537, 7 * full + 3):
            if ((count + r - 1) // r) * (r - 1) > count or (r - 1) > count:
                continue  # the algorithm itself falls back to radix 2 there (allreduce_sra.c:496-500)
            segs = sorted(mc.sra_segment(count, rank, r, size) for rank in range(full))
            pos = 0
            for off, ln in segs:
                assert off == pos, (r, size, count, segs)
                pos += ln
            assert pos == count
            for rank in range(full, size):   # extra ranks: whole vector
                assert mc.sra_segment(count, rank, r, size) == (0, count)


def test_run_rejects_bad_parameters():
    from xccl_amd.types import Dt, Op, Status
    lib = mc.replay_lib()
    assert lib.xccl_replay_run(None, None, 0) == Status.ERR_INVALID_PARAM
    arr = (ctypes.c_void_p * 2)(1, 2)
    for kw in (dict(team_size=1), dict(radix=1), dict(root=2), dict(dtype=int(Dt.UNSUPPORTED)), dict(alg=9)):
        base = dict(alg=0, reduce_mode=0, team_size=2, radix=2, root=0, count=4, dtype=int(Dt.INT32), op=int(Op.SUM))
        base.update(kw)
        prm = mc.ReplayParams(base["alg"], base["reduce_mode"], base["team_size"], base["radix"], base["root"],
                              base["count"], base["dtype"], base["op"],
                              ctypes.cast(arr, ctypes.POINTER(ctypes.c_void_p)),
                              ctypes.cast(arr, ctypes.POINTER(ctypes.c_void_p)))
        assert lib.xccl_replay_run(ctypes.byref(prm), None, 0) == Status.ERR_INVALID_PARAM, kw
