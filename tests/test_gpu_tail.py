"""The launch that walks the small rounds near the roots (cavs_treelstm_tail_fwd / _bwd) against
the per-round launches it replaces: same arithmetic in the same order, so every output must be
equal bit for bit; and the bounded wait of its barrier, made to give up from the host."""
import numpy as np
import pytest

from cavs_amd import hip, synth

pytestmark = pytest.mark.gpu

H = 512


@pytest.fixture(scope="module")
def g():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"
    import gpuutil

    hip.call("cavs_init", 0)
    return gpuutil


@pytest.fixture(autouse=True)
def _release_device_temporaries(g):
    yield
    g.release()


def rng(seed):
    return synth.SplitMix64(seed)


def packed_weights(g, U):
    """(row-major U on the device, its tile-major copy, the tile-major copy of the transposes)"""
    d_U, Upk, UTp = g.devf(U), g.zeros(4 * H * H), g.zeros(4 * H * H)
    T = hip.Task
    at = 4 * 3 * H * H
    jobs = [T(hip.TASK_SGD_PACK, 0.0, H, 3 * H, 0, g.P(Upk), g.P(d_U), None, None),
            T(hip.TASK_SGD_PACK, 0.0, H, H, 0, g.P(Upk) + at, g.P(d_U) + at, None, None),
            T(hip.TASK_PACK_T, 0.0, H, 3 * H, 0, g.P(UTp), g.P(d_U), None, None),
            T(hip.TASK_PACK_T, 0.0, H, H, 0, g.P(UTp) + at, g.P(d_U) + at, None, None)]
    g.call("cavs_run_tasks", len(jobs), (T * len(jobs))(*jobs), g.stream())
    return d_U, Upk, UTp


def forest(r, base, sizes):
    """A batch whose first `base` slab rows are earlier rounds and whose rounds of `sizes` vertices
    follow; every vertex of those rounds takes two children among the rows of earlier rounds that
    nobody has taken yet (now and then none).  Returns (offsets, child [2N])."""
    offs, N = [], base
    for n in sizes:
        offs.append(N)
        N += n
    child = np.full(2 * N, -1, np.int32)
    free = list(np.argsort(r.bulk_normal(base)))
    for off, n in zip(offs, sizes):
        for b in range(off, off + n):
            for side in range(2):
                if free and (b + side) % 11 != 5:
                    child[2 * b + side] = free.pop(int(r.bulk_uniform(1)[0] * len(free)))
        free.extend(range(off, off + n))  # this round's rows can be children from the next round on
    return offs, child, N


def chunks(offs, sizes):
    """the rounds as slices of at most 32 rows"""
    for off, n in zip(offs, sizes):
        for c0 in range(0, n, 32):
            yield off + c0, min(32, n - c0)


def sync_block(g):
    return g.dev(np.zeros(hip.lib().cavs_tail_sync_bytes() // 4, np.int32))


def plan_groups(offs, sizes, child, ngroups, backward=False):
    """Deals the rows of the rounds (first slab rows `offs`, `sizes` rows each, in the order they
    run) to `ngroups` groups, whole trees of the message flow among those rows per group, and
    returns (rows, nrounds [8], start, count, flags, max lists per group) as the tail entry points
    take them.  A group's share of a round goes into lists of at most 32 rows: the first waits for
    the group's earlier rounds, the last is an arrival."""
    R = len(sizes)
    lo = min(offs)
    comp = {}
    order = sorted(range(R), key=lambda k: offs[k], reverse=True)  # parents before children
    ncomp = 0
    for k in order:
        for b in range(offs[k], offs[k] + sizes[k]):
            if b not in comp:
                comp[b] = ncomp
                ncomp += 1
            for side in range(2):
                c = int(child[2 * b + side])
                if c >= lo:
                    comp[c] = comp[b]
    group_of = [c % ngroups for c in range(ncomp)]
    lists = [[] for _ in range(8)]  # per group: (rows, flags)
    for gi in range(ngroups):
        arrived = 0
        for k in range(R):
            mine = [b for b in range(offs[k], offs[k] + sizes[k]) if group_of[comp[b]] == gi]
            for c0 in range(0, len(mine), 32):
                last = c0 + 32 >= len(mine)
                lists[gi].append((mine[c0: c0 + 32], ((arrived if c0 == 0 else 0) << 1) | int(last)))
            arrived += 1 if mine else 0
    maxr = max(1, max(len(l) for l in lists))
    rows, nrounds = [], np.zeros(8, np.int32)
    start, count, flags = np.zeros(8 * maxr, np.int32), np.zeros(8 * maxr, np.int32), np.zeros(8 * maxr, np.int32)
    for gi in range(8):
        nrounds[gi] = len(lists[gi])
        for i, (mine, fl) in enumerate(lists[gi]):
            start[gi * maxr + i], count[gi * maxr + i], flags[gi * maxr + i] = len(rows), len(mine), fl
            rows.extend(mine)
    return np.asarray(rows, np.int32), nrounds, start, count, flags, maxr


@pytest.mark.parametrize("sizes,base,ngroups", [((30, 22, 13, 6, 3, 1, 1), 300, 1), ((32, 32, 17), 200, 1), ((5,), 40, 1), ((1, 1, 1, 1), 9, 8),
                                                ((16, 8, 4, 4, 2, 2, 1), 64, 3), ((166, 111, 76, 60, 43, 30, 22, 13, 6, 3, 1, 1), 700, 8),
                                                ((30, 22, 13, 6, 3, 1, 1), 300, 8), ((100, 70, 33, 5), 400, 1), ((425, 252, 166, 111, 76, 40, 9, 2), 1300, 8)])
def test_forward_tail_equals_the_per_round_launches_bit_for_bit(g, sizes, base, ngroups):
    r = rng(1000 * len(sizes) + sum(sizes))
    U = (r.bulk_normal(4 * H * H) / np.sqrt(H)).astype(np.float32)
    d_U, Upk, _ = packed_weights(g, U)
    offs, child, N = forest(r, base, sizes)
    pair = np.arange(N, dtype=np.int32)  # the message of slab row b goes to pool row b
    pair[offs[-1]] = -1                  # a root
    out_rows = np.argsort(r.bulk_normal(N)).astype(np.int32)
    pool0 = (r.bulk_normal(N * 2 * H).reshape(N, 2 * H) * 0.5).astype(np.float32)
    d_child, d_pair, d_out = g.devi(child), g.devi(pair), g.devi(out_rows)
    d_xW, d_bias = g.devf(r.bulk_normal(N * 4 * H)), g.devf(r.bulk_normal(4 * H) * 0.1)
    rows, nrounds, start, count, flags, maxr = plan_groups(offs, sizes, child, ngroups)
    assert count.max() <= 32
    d_tail_rows, flags_ptr = g.devi(rows), flags.ctypes.data
    outs = []
    for tail in (False, True):
        pool = g.devf(pool0)
        G, hlr, gates, msg, go = (g.zeros(2 * N, 2 * H, fill=-5.0), g.zeros(N, H, fill=-5.0), g.zeros(N, 6 * H, fill=-5.0),
                                  g.zeros(N, 2 * H, fill=-5.0), g.zeros(N, H, fill=-5.0))
        if tail:
            sync = sync_block(g)
            g.call("cavs_treelstm_tail_fwd", g.P(pool), g.P(d_child), g.P(d_pair), g.P(d_xW), 4 * H, g.P(Upk), g.P(d_bias), g.P(G),
                   g.P(hlr), g.P(gates), g.P(msg), g.P(go), g.P(d_out), g.P(d_tail_rows), ngroups, nrounds.ctypes.data, start.ctypes.data,
                   count.ctypes.data, flags_ptr, maxr, H, g.P(sync), 1 << 20, 0, g.stream())
            assert not g.host(sync).any(), "sync words after a completed launch"
        else:
            # (a round of more than 32 rows as slices of at most 32: the per-round launch then runs on
            # the tiles of four rows the tail launch computes with -- larger launches use tiles of
            # sixteen rows, whose sums come out in another order; a row's result does not depend on
            # the rows launched with it)
            for off, n in chunks(offs, sizes):
                g.call("cavs_treelstm_round_fwd_packed", g.P(pool), g.P(d_child) + 4 * 2 * off, g.P(d_pair) + 4 * off,
                       g.P(d_xW) + 4 * off * 4 * H, 4 * H, g.P(d_U), g.P(Upk), g.P(d_bias), g.P(G) + 4 * 2 * off * 2 * H,
                       g.P(hlr) + 4 * off * H, g.P(gates) + 4 * off * 6 * H, g.P(msg) + 4 * off * 2 * H, g.P(go), g.P(d_out) + 4 * off, n, H,
                       g.stream())
        outs.append([g.host(t) for t in (pool, G, hlr, gates, msg, go)])
    for a, b, what in zip(outs[0], outs[1], ("pool", "G", "hlr", "gates", "msg", "graph_out")):
        np.testing.assert_array_equal(a, b, err_msg=what)
    # the rounds did run and fed each other: the last round's gates are written and differ from the fill
    assert (outs[1][3][offs[-1]:] != -5.0).all()
    if len(sizes) > 1:
        assert (outs[1][0][offs[0]:offs[-1]] != pool0[offs[0]:offs[-1]]).any()


@pytest.mark.parametrize("sizes,base,leaves,ngroups", [((1, 1, 3, 6, 13, 22, 30), 300, 200, 1), ((17, 32, 32), 200, 120, 1), ((5,), 40, 40, 1),
                                                      ((1, 1, 1, 1), 9, 5, 8), ((1, 2, 2, 4, 4, 8, 16), 64, 30, 3),
                                                      ((1, 1, 3, 6, 13, 22, 30, 43, 60, 76, 111, 166), 700, 400, 8),
                                                      ((1, 1, 3, 6, 13, 22, 30), 300, 200, 8), ((5, 33, 70, 100), 400, 200, 1),
                                                      ((2, 9, 40, 76, 111, 166, 252, 425), 1300, 800, 8)])
def test_backward_tail_equals_the_per_round_launches_bit_for_bit(g, sizes, base, leaves, ngroups):
    """`sizes` lists the rounds in the order the backward pass runs them (roots first); in slab
    order they are the last rounds of the batch, smallest last."""
    r = rng(2000 * len(sizes) + sum(sizes))
    U = (r.bulk_normal(4 * H * H) / np.sqrt(H)).astype(np.float32)
    _, _, UTp = packed_weights(g, U)
    fwd_sizes = tuple(reversed(sizes))
    offs_f, kids, N = forest(r, base, fwd_sizes)
    offs = list(reversed(offs_f))
    gates = np.tanh(r.bulk_normal(N * 6 * H).reshape(N, 6 * H)).astype(np.float32)
    G = (r.bulk_normal(2 * N * 2 * H).reshape(2 * N, 2 * H) * 0.5).astype(np.float32)
    dret_rows = np.argsort(r.bulk_normal(N)).astype(np.int32)
    d_gates, d_G, d_dgo, d_rows, d_kids = g.devf(gates), g.devf(G), g.devf(r.bulk_normal(N * H)), g.devi(dret_rows), g.devi(kids)
    taken = set(int(k) for k in kids if k >= 0)
    orphans = np.array([v for v in range(N) if v not in taken], np.int32)  # nobody's child: their gradients come first
    d_orph = g.devi(orphans)
    rows, nrounds, start, count, flags, maxr = plan_groups(offs, sizes, kids, ngroups, backward=True)
    assert count.max() <= 32
    d_tail_rows, flags_ptr = g.devi(rows), flags.ctypes.data
    outs = []
    for tail in (False, True):
        dxW, dF, dc = g.zeros(N, 4 * H, fill=-3.0), g.zeros(2 * N, H, fill=-3.0), g.zeros(N, H, fill=-3.0)
        g.call("cavs_treelstm_bwd_gates_rows", g.P(d_orph), len(orphans), g.P(d_dgo), g.P(d_rows), g.P(d_gates), g.P(d_G), g.P(dxW),
               4 * H, g.P(dF), g.P(dc), leaves, H, g.stream())
        if tail:
            sync = sync_block(g)
            g.call("cavs_treelstm_tail_bwd", g.P(dxW), 4 * H, g.P(dF), g.P(dc), g.P(UTp), g.P(d_kids), g.P(d_gates), g.P(d_G), g.P(d_dgo),
                   g.P(d_rows), leaves, g.P(d_tail_rows), ngroups, nrounds.ctypes.data, start.ctypes.data, count.ctypes.data, flags_ptr, maxr, H,
                   g.P(sync), 1 << 20, 0, g.stream())
            assert not g.host(sync).any(), "sync words after a completed launch"
        else:
            for off, n in chunks(offs, sizes):
                g.call("cavs_treelstm_round_bwd_children_gates_packed", g.P(dxW), 4 * H, g.P(dF), g.P(dc), g.P(UTp),
                       g.P(d_kids) + 4 * 2 * off, g.P(d_gates), g.P(d_G), g.P(d_dgo), g.P(d_rows), off, n, leaves, H, g.stream())
        outs.append((g.host(dxW), g.host(dF), g.host(dc)))
    for a, b, what in zip(outs[0], outs[1], ("dxW", "dF", "dc")):
        np.testing.assert_array_equal(a, b, err_msg=what)
    kid_rows = sorted(taken)
    assert (outs[1][0][kid_rows] != -3.0).all()


def test_a_wait_that_cannot_complete_gives_up_and_every_wave_leaves(g):
    """extra_arrivals = 1: every wait expects one arrival more than there are workgroups, so the
    first wait runs into its bound.  The launch must end by itself with the status word set; after
    the caller clears the block the next launch works."""
    r = rng(77)
    sizes, base = (9, 4, 2), 40
    U = (r.bulk_normal(4 * H * H) / np.sqrt(H)).astype(np.float32)
    d_U, Upk, _ = packed_weights(g, U)
    offs, child, N = forest(r, base, sizes)
    pair = np.arange(N, dtype=np.int32)
    d_child, d_pair, d_out = g.devi(child), g.devi(pair), g.devi(np.arange(N, dtype=np.int32))
    d_xW, d_bias = g.devf(r.bulk_normal(N * 4 * H)), g.devf(np.zeros(4 * H))
    pool0 = (r.bulk_normal(N * 2 * H).reshape(N, 2 * H) * 0.5).astype(np.float32)
    rows, nrounds, start, count, _, maxr = plan_groups(offs, sizes, child, 2)
    d_tail_rows = g.devi(rows)

    def run(sync, extra, spins):
        pool = g.devf(pool0)
        G, hlr, gates = g.zeros(2 * N, 2 * H), g.zeros(N, H), g.zeros(N, 6 * H)
        g.call("cavs_treelstm_tail_fwd", g.P(pool), g.P(d_child), g.P(d_pair), g.P(d_xW), 4 * H, g.P(Upk), g.P(d_bias), g.P(G), g.P(hlr),
               g.P(gates), None, None, None, g.P(d_tail_rows), 2, nrounds.ctypes.data, start.ctypes.data, count.ctypes.data, None, maxr, H,
               g.P(sync), spins, extra, g.stream())
        return g.host(pool), g.host(gates)

    sync = sync_block(g)
    run(sync, 1, 200)
    words = g.host(sync)
    assert words[1] == 1, "the status word must say CAVS_TAIL_TIMEOUT"
    sync.zero_()
    pool_a, gates_a = run(sync, 0, 1 << 20)
    assert not g.host(sync).any()
    # and equals the per-round launches
    pool = g.devf(pool0)
    G, hlr, gates = g.zeros(2 * N, 2 * H), g.zeros(N, H), g.zeros(N, 6 * H)
    for off, n in zip(offs, sizes):
        g.call("cavs_treelstm_round_fwd_packed", g.P(pool), g.P(d_child) + 4 * 2 * off, g.P(d_pair) + 4 * off, g.P(d_xW) + 4 * off * 4 * H,
               4 * H, g.P(d_U), g.P(Upk), g.P(d_bias), g.P(G) + 4 * 2 * off * 2 * H, g.P(hlr) + 4 * off * H, g.P(gates) + 4 * off * 6 * H,
               None, None, None, n, H, g.stream())
    np.testing.assert_array_equal(pool_a, g.host(pool))
    np.testing.assert_array_equal(gates_a, g.host(gates))


def test_tail_entry_points_reject_what_they_cannot_run():
    assert hip.lib().cavs_tail_rounds_ok(32, 512) == 1 and hip.lib().cavs_tail_rounds_ok(33, 512) == 0
    assert hip.lib().cavs_tail_rounds_ok(8, 1024) == 0 and hip.lib().cavs_tail_rounds_ok(0, 512) == 0
    one, zero, big = np.asarray([1], np.int32), np.asarray([0], np.int32), np.asarray([40], np.int32)
    with pytest.raises(hip.CavsError, match="1..32 rows"):
        hip.call("cavs_treelstm_tail_fwd", 16, 16, 16, 16, 4 * H, 16, 16, 16, 16, 16, None, None, None, 16, 1, one.ctypes.data, zero.ctypes.data,
                 big.ctypes.data, None, 1, H, 16, 10, 0, None)
    waits = np.asarray([2], np.int32)  # the only list waits for an arrival nobody makes
    with pytest.raises(hip.CavsError, match="waits for 1 arrivals"):
        hip.call("cavs_treelstm_tail_fwd", 16, 16, 16, 16, 4 * H, 16, 16, 16, 16, 16, None, None, None, 16, 1, one.ctypes.data, zero.ctypes.data,
                 one.ctypes.data, waits.ctypes.data, 1, H, 16, 10, 0, None)
    with pytest.raises(hip.CavsError, match="H = 512"):
        hip.call("cavs_treelstm_tail_bwd", 16, 4 * 256, 16, 16, 16, 16, 16, 16, 16, 16, 0, 16, 1, one.ctypes.data, zero.ctypes.data,
                 one.ctypes.data, None, 1, 256, 16, 10, 0, None)
    with pytest.raises(hip.CavsError, match="1..8 groups"):
        hip.call("cavs_treelstm_tail_bwd", 16, 4 * H, 16, 16, 16, 16, 16, 16, 16, 16, 0, 16, 9, one.ctypes.data, zero.ctypes.data,
                 one.ctypes.data, None, 1, H, 16, 10, 0, None)


@pytest.mark.parametrize("pairing", ["rowid", "reference"])
def test_a_training_step_is_the_same_with_and_without_the_tail_launches(g, pairing):
    """The engine on a batch of parse trees at H = 512, one launch per round against the rounds near
    the roots inside tail launches.  With at most 4 rows per group and round the launches take the
    rounds of at most 32 vertices, which the per-round launches also run on tiles of four rows: loss,
    outputs and every gradient bit for bit (the embedding gradient, whose repeated rows are added
    with atomics, to the tolerance).  With the default limit they reach rounds the per-round
    launches run on tiles of sixteen rows (another order of the same sums): to the tolerance."""
    from cavs_amd import session
    from tolerance import close

    w = synth.make_workload("C3", B=24)
    assert w["H"] == H
    res = {}
    for tail_rows in (-1, 4, 0):
        s = session.Session("treelstm", H=w["H"], E=w["E"], V=w["V"], C_=w["C"], pairing=pairing, tail_rows=tail_rows)
        s.set_params(w["params"])
        steps = []
        for _ in range(2):  # the second step reads the weights the first one updated and packed
            s.step(w["graph"], w["x"], w["labels"], backward=True, lr=0.05)
            steps.append((s.fetch("loss"), s.fetch("graph_out"), s.grads()))
        res[tail_rows] = (steps, s.counter("tail_rounds"), s.counter("launches"))
        if tail_rows >= 0:
            assert s.counter("tail_ready") == 1, "the device did not pass the probe of the tail launches"
        s.close()
    (steps0, used0, n0), (steps4, used4, n4), (steps1, used1, n1) = res[-1], res[4], res[0]
    assert used0 == 0
    assert used4 >= 4 and n4 < n0, "the tail launches did not run"
    assert used1 >= used4 and n1 <= n4
    (l0, g0, gr0), (l4, g4, gr4) = steps0[0], steps4[0]
    np.testing.assert_array_equal(l0, l4)
    np.testing.assert_array_equal(g0, g4)
    for k in gr0:
        if k == "dEmb":
            close(gr4[k], gr0[k].astype(np.float64), k)
        else:
            np.testing.assert_array_equal(gr0[k], gr4[k], err_msg=k)
    # the second step starts from an embedding table updated with a gradient whose last bits depend
    # on the order of its atomics; the default limit changes the order of sums in the larger rounds
    for (la, ga, gra), (lb, gb, grb), what in ((steps0[1], steps4[1], "second step, 4 rows per group"), (steps0[0], steps1[0], "first step"),
                                              (steps0[1], steps1[1], "second step")):
        close(lb, la.astype(np.float64), "loss, " + what)
        close(gb, ga.astype(np.float64), "graph_out, " + what)
        for k in gra:
            close(grb[k], gra[k].astype(np.float64), k + ", " + what)


def test_the_device_built_schedule_runs_the_tail_launches_too(g):
    """schedule="device": the children-by-slab-row list comes back from the device scheduler, the host
    deals its trees to the groups and the row lists go up; the step is the one of the host scheduler
    (same plan, same launches) bit for bit, apart from the embedding gradient's atomics."""
    from cavs_amd import session
    from tolerance import close

    w = synth.make_workload("C3", B=24)
    res = {}
    for schedule in ("host", "device"):
        s = session.Session("treelstm", H=w["H"], E=w["E"], V=w["V"], C_=w["C"], schedule=schedule)
        s.set_params(w["params"])
        s.step(w["graph"], w["x"], w["labels"], backward=True, lr=0.0)
        res[schedule] = (s.fetch("loss"), s.fetch("graph_out"), s.grads(), s.counter("tail_rounds"), s.counter("launches"),
                         s.counter("tail_first_round"), s.counter("scheduler"))
        s.close()
    h, d = res["host"], res["device"]
    assert d[6] == 1 and h[6] == 0
    assert d[3] == h[3] > 0 and d[5] == h[5], "the device-scheduled step did not run the same tail launches"
    np.testing.assert_array_equal(d[0], h[0])
    np.testing.assert_array_equal(d[1], h[1])
    for k in h[2]:
        if k == "dEmb":
            close(d[2][k], h[2][k].astype(np.float64), k)
        else:
            np.testing.assert_array_equal(d[2][k], h[2][k], err_msg=k)


def test_a_guarded_launch_of_jobs_runs_only_while_the_watched_word_is_zero(g):
    """CAVS_TASK_GUARD: the parameter updates of a step watch the status word of the tail launches."""
    T = hip.Task
    w0 = np.arange(1000, dtype=np.float32)
    grad = np.ones(1000, np.float32)
    d_w, d_g, flag = g.devf(w0), g.devf(grad), g.dev(np.zeros(4, np.int32))
    jobs = [T(hip.TASK_GUARD, 0.0, 0, 0, 0, g.P(flag) + 4, None, None, None), T(hip.TASK_SGD, 0.5, 1000, 0, 0, g.P(d_w), g.P(d_g), None, None)]
    g.call("cavs_run_tasks", 2, (T * 2)(*jobs), g.stream())
    np.testing.assert_array_equal(g.host(d_w), w0 - 0.5)
    flag[1] = 1
    g.call("cavs_run_tasks", 2, (T * 2)(*jobs), g.stream())
    np.testing.assert_array_equal(g.host(d_w), w0 - 0.5)  # untouched
    flag[1] = 0
    g.call("cavs_run_tasks", 2, (T * 2)(*jobs), g.stream())
    np.testing.assert_array_equal(g.host(d_w), w0 - 1.0)
    with pytest.raises(hip.CavsError, match="one guard"):
        g.call("cavs_run_tasks", 2, (T * 2)(jobs[0], jobs[0]), g.stream())
