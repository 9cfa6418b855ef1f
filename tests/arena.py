"""The per-step index lists the kernels consume (t2j, pair, child, kid_rows, roots, orphans),
derived from a scheduler trace (the oracle's): the expected value of whatever builds them in the
product -- the host scheduler's upload or the device scheduler."""
import numpy as np


def expected_arena(trace, graph, nch, pairing):
    """trace: oracle.sched_trace(graph).  Returns dict of int arrays."""
    N = trace["N"]
    t2j = np.array(trace["tids_to_jobids"], np.int64)
    pair = np.full(N, -1, np.int64)
    child = np.full(nch * N, -1, np.int64)
    for rd in trace["fwd"]:
        off = rd["offset"]
        for b, t in enumerate(rd["scatter"][0]):
            if pairing == "reference":   # b-th list entry with b-th slab row of the round
                pair[off + b] = t
            else:
                pair[t] = t
        for c in range(nch):
            for b, t in enumerate(rd["gather"][c]):
                child[nch * (off + b) + c] = t
    parents, off = [], 0
    for row in graph:
        n = int(np.argmax(row == -1)) + 1
        parents += [off + int(p) if p >= 0 else -1 for p in row[:n]]
        off += n
    roots = np.array([v for v, p in enumerate(parents) if p < 0], np.int64)
    inv = np.full(N, -1, np.int64)
    for v in range(N):
        if pair[v] >= 0:
            assert inv[pair[v]] < 0
            inv[pair[v]] = v
    kid = np.where(child >= 0, inv[np.maximum(child, 0)], -1)
    orphans = np.array([v for v in range(N) if pair[v] < 0], np.int64)
    r2o = np.array(trace["round2offset"], np.int64)
    return dict(N=N, R=len(trace["fwd"]), t2j=t2j, pair=pair, child=child, kid=kid, roots=roots, orphans=orphans,
                round2offset=r2o)
