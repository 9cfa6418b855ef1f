"""Pins the scheduler restatement (oracle/sched.c) without retyping it:
hand-derived known answers, structural invariants, and an independent
level/positional formulation of the batching order."""
import json
import os

import numpy as np
import pytest

from cavs_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "sched_kat.json")))["cases"]


@pytest.mark.parametrize("case", KATS, ids=[c["name"] for c in KATS])
def test_hand_derived_known_answers(oracle, case):
    tr = oracle.sched_trace(np.array(case["graph"], np.int32))
    assert tr["N"] == case["N"]
    assert tr["round2offset"] == case["round2offset"]
    assert tr["tids_to_jobids"] == case["tids_to_jobids"]
    assert tr["fwd"] == case["fwd"]
    assert tr["bwd"] == case["bwd"]


def _adjacency(graph):
    """independent parse of the parent-array wire format"""
    parents, offs, off = [], [], 0
    for row in graph:
        n = int(np.argmax(row == -1)) + 1
        offs.append(off)
        parents += [off + int(p) if p >= 0 else -1 for p in row[:n]]
        off += n
    children = [[] for _ in parents]
    for v, p in enumerate(parents):
        if p >= 0:
            children[p].append(v)
    return parents, children


def _independent_schedule(graph):
    """Level of a vertex = 1 + max level of its children; within a level the
    order is the order in which the last child of each vertex appears in the
    previous level (a different algorithm from the reference's counters)."""
    parents, children = _adjacency(graph)
    n = len(parents)
    level = [0] * n
    for v in range(n):  # children have smaller... not guaranteed: iterate to a fixed point
        pass
    changed = True
    while changed:
        changed = False
        for v in range(n):
            if children[v]:
                l = 1 + max(level[c] for c in children[v])
                if l != level[v]:
                    level[v], changed = l, True
    rounds = [[v for v in range(n) if level[v] == 0 and parents[v] >= 0]]
    while True:
        pos = {v: i for i, v in enumerate(rounds[-1])}
        r = len(rounds)
        cand = [v for v in range(n) if level[v] == r]
        if not cand:
            break
        key = {v: max(pos[c] for c in children[v] if level[c] == r - 1) for v in cand}
        rounds.append(sorted(cand, key=lambda v: key[v]))
    return parents, children, rounds


def _random_graphs():
    out = []
    for seed in range(12):
        g, _, _ = synth.tree_batch(100 + seed, 1 + seed % 7, 2, 9 + seed)
        out.append(g)
    for seed in range(6):
        g, _, _ = synth.chain_batch(200 + seed, 2 + seed, 2, 12)
        out.append(g)
    return out


@pytest.mark.parametrize("idx", range(18))
def test_batch_schedule_matches_independent_formulation(oracle, idx):
    graph = _random_graphs()[idx]
    parents, children, rounds = _independent_schedule(graph)
    tr = oracle.sched_trace(graph)
    assert [r["exec"] for r in tr["fwd"]] == rounds
    # tensor ids: exclusive prefix of round sizes, row index == position
    offs = np.concatenate([[0], np.cumsum([len(r) for r in rounds])]).tolist()
    assert tr["round2offset"] == offs
    t2j = [v for r in rounds for v in r]
    assert tr["tids_to_jobids"][: len(t2j)] == t2j
    j2t = {v: t for t, v in enumerate(t2j)}
    for r, rd in enumerate(tr["fwd"]):
        assert rd["offset"] == offs[r]
        if r == 0:
            assert rd["gather"] == [[], []]
            assert rd["gather_init"] == rounds[0]
        else:
            for c in range(2):
                want = [j2t[children[v][c]] for v in rd["exec"] if len(children[v]) > c]
                assert rd["gather"][c] == want
        # scatter list: tensor ids of the non-root jobs, in job order
        assert rd["scatter"][0] == [j2t[v] for v in rd["exec"] if parents[v] >= 0]
        assert rd["scatter"][1] == []
    # backward = forward replayed in reverse with the lists swapped
    assert len(tr["bwd"]) == len(tr["fwd"])
    roots = [j2t[v] for r in rounds for v in r if parents[v] < 0]
    for rb, rf in zip(tr["bwd"], reversed(tr["fwd"])):
        assert rb["exec"] == rf["exec"] and rb["offset"] == rf["offset"]
        assert rb["gather"][0] == rf["scatter"][0]
        assert rb["scatter"] == rf["gather"]
        assert rb["gather_init"] == roots


@pytest.mark.parametrize("idx", range(18))
def test_schedule_invariants(oracle, idx):
    graph = _random_graphs()[idx]
    parents, children, _ = _independent_schedule(graph)
    tr = oracle.sched_trace(graph)
    n = tr["N"]
    assert n == synth.total_length(graph)
    assert sorted(tr["tids_to_jobids"]) == list(range(n))  # a permutation (no singletons here)
    done = set()
    for rd in tr["fwd"]:
        for v in rd["exec"]:
            assert all(c in done for c in children[v])  # children strictly earlier
        done.update(rd["exec"])
    assert len(done) == n


@pytest.mark.parametrize("idx", range(18))
def test_serial_schedule(oracle, idx):
    """SerialGraphScheduler: one vertex per round, tensor id == vertex id, samples
    in order, a valid topological order (graph_scheduler.cc:83-167)."""
    graph = _random_graphs()[idx]
    parents, children, _ = _independent_schedule(graph)
    tr = oracle.sched_trace(graph, batching=False)
    order = [r["exec"][0] for r in tr["fwd"]]
    assert sorted(order) == list(range(tr["N"]))
    seen = set()
    for rd in tr["fwd"]:
        (v,) = rd["exec"]
        assert rd["offset"] == v
        assert all(c in seen for c in children[v])
        seen.add(v)
        assert rd["gather"] == [[c] for c in children[v]] + [[]] * (2 - len(children[v]))
        assert rd["scatter"][0] == ([v] if parents[v] >= 0 else [])
    # samples are processed one after the other
    sample_of = []
    for i, row in enumerate(graph):
        sample_of += [i] * (int(np.argmax(row == -1)) + 1)
    s = [sample_of[v] for v in order]
    assert s == sorted(s)
    # backward: roots first, children after their parent, scatter lists = children ids
    border = [r["exec"][0] for r in tr["bwd"]]
    assert sorted(border) == list(range(tr["N"]))
    seen = set()
    for rd in tr["bwd"]:
        (v,) = rd["exec"]
        assert parents[v] < 0 or parents[v] in seen
        seen.add(v)
        assert [l for l in rd["scatter"] if l] == [[c] for c in children[v]]
        assert rd["gather"][0] == ([v] if parents[v] >= 0 else [])


def test_same_shape_batches_scatter_is_identity(oracle):
    """For equal-shape samples no root precedes a non-root in any round, so the
    scatter list of a round is exactly its tensor-id range."""
    rng = synth.SplitMix64(7)
    tree = synth.random_binary_tree(rng, 9)
    graph = synth.pack_graph([tree] * 5, len(tree))
    tr = oracle.sched_trace(graph)
    for rd in tr["fwd"][:-1]:
        assert rd["scatter"][0] == list(range(rd["offset"], rd["offset"] + len(rd["exec"])))


def test_rejects_sample_without_terminator(oracle):
    import ctypes as C

    g = np.array([[1, 2, 0]], np.int32)
    out = np.zeros(64, np.int32)
    n = oracle.lib().or_sched_trace(g.ctypes.data_as(C.c_void_p), 1, 3, 1, 0,
                                    out.ctypes.data_as(C.c_void_p), 64)
    assert n == 0  # LoadGraph's length CHECK (graph_scheduler.cc:41)


@pytest.mark.parametrize("kind,seed,B,lo,hi", [("tree", 11, 5, 2, 9), ("tree", 12, 33, 2, 40), ("chain", 13, 9, 2, 30),
                                               ("tree", 14, 1, 7, 7)])
def test_batch_schedule_is_the_samples_schedules_merged_round_by_round(oracle, kind, seed, B, lo, hi):
    """What the device scheduler builds on: every round of a batch lists its vertices sample by
    sample, each sample's in the order that sample alone would produce them, so
    tensor id = round2offset[r] + (vertices of earlier samples in round r) + position in the
    sample's own round; and under the reference pairing slab row (tensor id - roots of earlier
    samples in the round) holds the message of a non-root vertex."""
    import arena

    graph = (synth.tree_batch if kind == "tree" else synth.chain_batch)(seed, B, lo, hi)[0]
    tr = oracle.sched_trace(graph)
    nch = 2 if kind == "tree" else 1
    want = arena.expected_arena(tr, graph, nch, "reference")
    singles = [oracle.sched_trace(graph[i:i + 1]) for i in range(B)]
    R = len(tr["fwd"])
    cnt = np.zeros((B, R + 1), np.int64)
    for s, st in enumerate(singles):
        for r, rd in enumerate(st["fwd"]):
            cnt[s, r] = len(rd["exec"])
    depth = [len(st["fwd"]) for st in singles]
    r2o = np.concatenate([[0], np.cumsum(cnt.sum(0))])
    assert r2o[: R + 1].tolist() == tr["round2offset"]
    soff = np.concatenate([[0], np.cumsum([st["N"] for st in singles])])
    t2j, pair = np.full(tr["N"], -1), np.full(tr["N"], -1)
    for s, st in enumerate(singles):
        for r, rd in enumerate(st["fwd"]):
            before = cnt[:s, r].sum()
            roots_before = sum(1 for q in range(s) if depth[q] - 1 == r)
            for i, v in enumerate(rd["exec"]):
                t = r2o[r] + before + i
                t2j[t] = soff[s] + v
                if r < depth[s] - 1:
                    pair[t - roots_before] = t
    assert t2j.tolist() == want["t2j"].tolist()
    assert pair.tolist() == want["pair"].tolist()
