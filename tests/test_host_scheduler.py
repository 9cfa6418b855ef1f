"""The production scheduler (cavs_amd/host/scheduler.cc) must expose bit-exactly the
rounds and index lists of the reference's schedulers.  Checked against the hand-derived
known answers and, over random batches, against the oracle.  Host only: no GPU."""
import functools
import json
import os

import numpy as np
import pytest

from cavs_amd import session, synth, hip

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "sched_kat.json")))["cases"]


@pytest.mark.parametrize("case", KATS, ids=[c["name"] for c in KATS])
def test_known_answers(case):
    tr = session.schedule_trace(np.array(case["graph"], np.int32))
    for k in ("N", "round2offset", "tids_to_jobids", "fwd", "bwd"):
        assert tr[k] == case[k], k


@functools.lru_cache(maxsize=None)
def _graphs():
    out = []
    for seed in range(10):
        out.append(synth.tree_batch(300 + seed, 1 + 3 * seed, 2, 5 + 6 * seed)[0])
    for seed in range(6):
        out.append(synth.chain_batch(400 + seed, 1 + 2 * seed, 2, 25)[0])
    out.append(synth.make_workload("C3")["graph"])
    out.append(synth.make_workload("C4")["graph"])
    return out


@pytest.mark.parametrize("idx", range(18))
@pytest.mark.parametrize("batching", [True, False])
def test_matches_oracle_bit_exact(oracle, idx, batching):
    graph = _graphs()[idx]
    want = oracle.sched_trace(graph, batching=batching)
    got = session.schedule_trace(graph, batching=batching)
    assert got["N"] == want["N"]
    assert got["tids_to_jobids"] == want["tids_to_jobids"]
    assert got["round2offset"] == want["round2offset"]
    assert len(got["fwd"]) == len(want["fwd"]) and len(got["bwd"]) == len(want["bwd"])
    for a, b in zip(got["fwd"] + got["bwd"], want["fwd"] + want["bwd"]):
        assert a == b


def test_rejects_malformed_feeds():
    with pytest.raises(hip.CavsError, match="terminator"):
        session.schedule_trace(np.array([[1, 2, 0]], np.int32))
    with pytest.raises(hip.CavsError, match="out of range"):
        session.schedule_trace(np.array([[5, -1, -1]], np.int32))
    with pytest.raises(hip.CavsError, match="3 children"):
        session.schedule_trace(np.array([[3, 3, 3, -1]], np.int32))
    with pytest.raises(hip.CavsError, match="single-vertex"):
        session.index_lists(np.array([[-1, -1], [1, -1]], np.int32), 1)
    with pytest.raises(hip.CavsError, match="cycle"):   # vertices 0 and 1 are each other's parent
        session.schedule_trace(np.array([[1, 0, 3, -1]], np.int32))
    with pytest.raises(hip.CavsError, match="cycle"):   # a vertex that is its own parent
        session.schedule_trace(np.array([[0, 2, -1]], np.int32))


@pytest.mark.parametrize("idx", range(18))
@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_index_lists_match_the_oracles_schedule_and_invert(oracle, idx, pairing):
    """The lists the kernels consume (one entry per slab row) against the oracle's per-round
    lists, and back: the lists alone determine the complete schedule."""
    import arena

    graph = _graphs()[idx]
    tr = oracle.sched_trace(graph)
    nch = 2 if any(rd["gather"][1] for rd in tr["fwd"]) else 1
    want = arena.expected_arena(tr, graph, nch, pairing)
    got = session.index_lists(graph, nch, pairing)
    assert got["N"] == want["N"]
    for k in ("t2j", "pair", "child", "roots", "kid", "orphans"):
        assert got[k].tolist() == want[k].tolist(), k
    B, maxlen = graph.shape
    back = session.trace_from_lists(B, maxlen, nch, tr["round2offset"], got["t2j"], got["pair"], got["child"], got["roots"])
    assert back == session.schedule_trace(graph) == tr


def test_index_lists_refuse_mixed_arity_and_report_non_forests():
    with pytest.raises(hip.CavsError, match="mixes"):    # a chain inside a binary vertex function
        session.index_lists(np.array([[1, 2, -1]], np.int32), 2)
    with pytest.raises(hip.CavsError, match="two children"):
        session.index_lists(np.array([[2, 2, -1]], np.int32), 1)
    g = synth.tree_batch(7, 9, 2, 20)[0]
    assert session.index_lists(g, 2)["kid"] is not None
    assert session.index_lists(g, 2, fused_limit=3)["kid"] is None   # a round with children above the limit


def _check_tail_lists(graph, pairing, rows_limit, groups=8, max_lists=32):
    """Properties any deal must have, from the lists alone.  Returns the plan (or None)."""
    t = session.tail_lists(graph, pairing, rows_limit=rows_limit, groups=groups, max_lists=max_lists)
    lists = session.index_lists(graph, 2, pairing)
    tr = session.schedule_trace(graph)
    r2o = tr["round2offset"]
    if t is None:
        return None
    N, kid = lists["N"], lists["kid"].reshape(-1, 2)
    first, M = t["first"], t["M"]
    lo = r2o[first]
    round_of = np.searchsorted(np.asarray(r2o), np.arange(N), side="right") - 1
    owner = np.full(N, -1)
    # the slab rows from round `first` on, each exactly once
    assert sorted(t["rows"].tolist()) == list(range(lo, N))
    assert 1 <= first and len(r2o) - 1 - first >= 2
    for g in range(groups):
        n = int(t["nrounds"][g])
        assert 0 <= n <= M <= max_lists
        arrived, done_rounds, prev_round = 0, 0, -1
        for i in range(n):
            s, c, f = int(t["start"][g, i]), int(t["count"][g, i]), int(t["flags"][g, i])
            assert 1 <= c <= 32
            rows = t["rows"][s:s + c]
            rd = set(round_of[rows].tolist())
            assert len(rd) == 1, "a list holds rows of one round"
            k = rd.pop()
            assert k >= prev_round, "forward order"
            if k != prev_round:   # first slice of the group's share of this round: waits for all its earlier rounds
                assert f >> 1 == arrived, (g, i, f, arrived)
            else:                 # a further slice of the same round: no wait
                assert f >> 1 == 0
            prev_round = k
            owner[rows] = g
            last_slice = i + 1 == n or round_of[t["rows"][int(t["start"][g, i + 1])]] != k
            assert (f & 1) == int(last_slice), "a round's last slice is its arrival"
            arrived += f & 1
        # the backward lists: the same slices, rounds in reverse
        fwd = [(int(t["start"][g, i]), int(t["count"][g, i])) for i in range(n)]
        bwd = [(int(t["bstart"][g, i]), int(t["bcount"][g, i])) for i in range(n)]
        assert sorted(fwd) == sorted(bwd)
        brounds = [int(round_of[t["rows"][s]]) for s, _ in bwd]
        assert brounds == sorted(brounds, reverse=True)
        barrived = 0
        for i in range(n):
            f = int(t["bflags"][g, i])
            new_round = i == 0 or brounds[i] != brounds[i - 1]
            assert f >> 1 == (barrived if new_round else 0)
            barrived += f & 1
    assert (owner[lo:] >= 0).all()
    # no message crosses groups: a row's children inside the suffix belong to its group
    for v in range(lo, N):
        for c in kid[v]:
            if c >= lo:
                assert owner[c] == owner[v], (v, c)
    # no group gets more than the limit of any round
    for k in range(first, len(r2o) - 1):
        for g in range(groups):
            assert int(((round_of[lo:] == k) & (owner[lo:] == g)).sum()) <= rows_limit
    return t


@pytest.mark.parametrize("pairing", ["reference", "rowid"])
@pytest.mark.parametrize("seed,B,lmin,lmax", [(11, 64, 2, 56), (12, 24, 2, 56), (13, 200, 8, 40), (14, 7, 2, 9)])
def test_the_deal_of_trees_to_the_groups_of_the_tail_launches(seed, B, lmin, lmax, pairing):
    """Whole trees of the message flow per group, every row of the suffix exactly once, a group's share
    of a round in slices of at most 32 rows, wait / arrive flags that match the slices, the backward
    lists the forward ones reversed by round, and the limits kept."""
    graph = synth.tree_batch(seed, B, lmin, lmax, 2 * lmax - 1)[0]
    for limit in (4, 32, 96):
        t = _check_tail_lists(graph, pairing, limit)
        if B >= 24:
            assert t is not None, "a batch of this size has rounds to deal"
    _check_tail_lists(graph, pairing, 32, groups=3)


def test_the_deal_starts_later_under_a_tighter_limit_and_refuses_what_does_not_fit():
    graph = synth.tree_batch(21, 64, 2, 56, 111)[0]
    a, b = session.tail_lists(graph, rows_limit=32), session.tail_lists(graph, rows_limit=4)
    assert a["first"] < b["first"]
    assert len(a["rows"]) > len(b["rows"])
    # two lists per group cannot hold three rounds or more
    assert session.tail_lists(graph, rows_limit=32, max_lists=1) is None
    # a chain batch has no binary rounds to deal
    chain = synth.chain_batch(5, 6, 4, 9, 9)[0]
    with pytest.raises(hip.CavsError):
        session.tail_lists(chain)
