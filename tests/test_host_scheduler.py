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
