"""End-to-end GPU parity: one forward+backward pass through the host runtime and the
HIP backend against the oracle on the same seeded inputs.  Schedule and index lists
bit-exact; fp32 losses, activations and gradients within 1e-4 relative / 1e-5 absolute of the
oracle's dataflow evaluated in double precision (tolerance.py), at every site."""
import numpy as np
import pytest

from cavs_amd import hip, session, synth
from test_oracle_models import small_workload
from tolerance import close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"


def run_both(oracle, w, *, loss="softmax", pairing="reference", batching=True, **kw):
    print(f"[case] model={w['model']} N={w['N']} H={w['H']} loss={loss} pairing={pairing} batching={batching}", flush=True)
    want = oracle.model_step(w["model"], w["graph"], w["x"], w["labels"], w["params"], H=w["H"], E=w["E"],
                             V=w["V"], Cc=w["C"], loss=loss, pairing=pairing, batching=batching, precise=True,
                             threads=16, **kw)
    s = session.Session(w["model"], H=w["H"], E=w["E"], V=w["V"], C_=w["C"], loss=loss, pairing=pairing,
                        opt=session.OPT_BATCHING if batching else 0, **kw)
    names = {"treelstm": ("Emb", "W", "U", "Bv"), "lstm": ("Emb", "W", "Bv"),
             "treefc": ("W", "Bv") if kw.get("use_bias") else ("W",)}[w["model"]]
    if loss == "softmax":
        names += ("Wfc", "bfc")
    s.set_params({k: w["params"][k] for k in names})
    s.step(w["graph"], w["x"], w["labels"], backward=True)
    got = dict(loss=s.fetch("loss"), graph_out=s.fetch("graph_out"), dgraph_out=s.fetch("dgraph_out"),
               msg_pool=s.fetch("msg_pool"), grads=s.grads(), trace=s.schedule_trace())
    s.close()
    return got, want


def compare(got, want, loss="softmax", **tol):
    """The softmax configurations (the headline among them) are held to the literal bar, 1e-4
    relative / 1e-5 absolute with no tensor-scale factor; the sum-of-squares and sum-of-magnitudes
    losses, whose weight gradients reach the tens, measure "absolute" in units of the tensor's
    largest entry (tolerance.py)."""
    if loss == "softmax":
        tol.setdefault("scaled", False)
    for k in ("loss", "graph_out", "dgraph_out"):
        close(got[k], want[k], k, **tol)
    # pool rows of roots are never written by any Scatter: their content is unspecified
    written = sorted({t for rd in got["trace"]["fwd"] for t in rd["scatter"][0]})
    close(got["msg_pool"][written], want["msg_pool"][written], "msg_pool", **tol)
    for k, v in want["grads"].items():
        if k in got["grads"]:
            close(got["grads"][k], v, k, **tol)


CASES = [("treelstm", dict()), ("lstm", dict()), ("treefc", dict(act=1, use_bias=True, use_x=True)),
         ("treefc", dict(act=0))]


@pytest.mark.parametrize("model,kw", CASES)
@pytest.mark.parametrize("pairing", ["reference", "rowid"])
@pytest.mark.parametrize("loss", ["softmax", "root_sq", "sum_abs"])
def test_small_skewed_batches(oracle, model, kw, pairing, loss):
    w = small_workload(model, 61, B=6, H=16, E=12)
    got, want = run_both(oracle, w, loss=loss, pairing=pairing, **kw)
    compare(got, want, loss=loss)
    assert got["trace"] == oracle.sched_trace(w["graph"])  # bit-exact lists on the running session


@pytest.mark.parametrize("model,kw", CASES)
def test_serial_scheduler(oracle, model, kw):
    w = small_workload(model, 62, B=3, H=8, E=8)
    got, want = run_both(oracle, w, batching=False, **kw)
    compare(got, want)
    assert got["trace"] == oracle.sched_trace(w["graph"], batching=False)


@pytest.mark.parametrize("model,kw", CASES)
def test_odd_sizes_take_the_unaligned_paths(oracle, model, kw):
    """hidden / embedding sizes that are not multiples of 4 (scalar loads everywhere)"""
    w = small_workload(model, 63, B=4, H=6, E=5, V=11, C=3)
    got, want = run_both(oracle, w, **kw)
    compare(got, want)


@pytest.mark.parametrize("name,scale", [("C1", 0.25), ("C2", 0.25), ("C3", 0.125), ("C4", 0.0625), ("C5", 0.0625)])
def test_benchmark_configs_scaled(oracle, name, scale):
    """The benchmark batches -- their own graphs, batch sizes (C4: 128 sequences, C5: 256 trees of up
    to 511 vertices, N ~ 72 k), vocabularies and class counts (C4: the 10000-way head) -- at reduced
    widths so that the oracle finishes in seconds."""
    w = synth.make_workload(name, scale=scale)
    kw, loss = {}, "softmax"
    if w["model"] == "treefc":
        kw, loss = dict(act=1, use_bias=True, use_x=True), "root_sq"
    got, want = run_both(oracle, w, loss=loss, **kw)
    compare(got, want, loss=loss)


@pytest.mark.parametrize("name", ["C1", "C2", "C3"])
def test_benchmark_configs_at_full_size(oracle, name):
    """The benchmark's own batches at their own widths against the oracle (it needs a second or
    two for these three; C4 and C5 meet it at their own batch sizes and reduced widths above, and
    at full size below), at the same 1e-4 relative / 1e-5 absolute bar as the small cases."""
    w = synth.make_workload(name)
    kw, loss = {}, "softmax"
    if w["model"] == "treefc":
        kw, loss = dict(act=1, use_bias=True, use_x=True), "root_sq"
    got, want = run_both(oracle, w, loss=loss, **kw)
    compare(got, want, loss=loss)


@pytest.mark.parametrize("name", ["C4", "C5"])
def test_benchmark_configs_at_full_size_against_recorded_values(name):
    """C4 and C5 at their full sizes.  The checker needs minutes for these in double precision, so
    its results were recorded once (tests/golden/make_fullsize_fixtures.py: per tensor the norm and
    512 entries at fixed positions); the GPU step is held to them at the literal bar, 1e-4 relative /
    1e-5 absolute."""
    import os

    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", f"fullsize_{name}.npz"))
    w = synth.make_workload(name)
    assert int(fx["N"]) == w["N"]
    print(f"[case] full size {name} N={w['N']} H={w['H']}", flush=True)
    s = session.Session(w["model"], H=w["H"], E=w["E"], V=w["V"], C_=w["C"], loss="softmax", pairing="reference")
    names = {"treelstm": ("Emb", "W", "U", "Bv"), "lstm": ("Emb", "W", "Bv")}[w["model"]] + ("Wfc", "bfc")
    s.set_params({k: w["params"][k] for k in names})
    s.step(w["graph"], w["x"], w["labels"], backward=True)
    got = dict(loss=s.fetch("loss"), graph_out=s.fetch("graph_out"), dgraph_out=s.fetch("dgraph_out"), **s.grads())
    s.close()
    checked = 0
    for k, v in got.items():
        if k + ".idx" not in fx:
            continue
        flat = np.asarray(v, np.float64).ravel()
        assert tuple(fx[k + ".shape"]) == tuple(np.shape(v)) or flat.size == int(np.prod(fx[k + ".shape"])), k
        close(flat[fx[k + ".idx"]], fx[k + ".val"], f"{name} {k} (recorded entries)", scaled=False)
        norm = float(np.sqrt((flat * flat).sum()))
        assert abs(norm - float(fx[k + ".norm"])) <= 1e-4 * float(fx[k + ".norm"]) + 1e-7, (k, norm, float(fx[k + ".norm"]))
        checked += 1
    assert checked >= 8, checked


@pytest.mark.parametrize("name,B", [("C4", 8), ("C5", 6)])
def test_benchmark_configs_at_full_width(oracle, name, B):
    """C4 and C5 at their own widths (H = 512 with the 10000-way head; E = H = 1024 with trees of up
    to 511 vertices) on a few samples of their batches, which is what the oracle can evaluate in
    double within seconds: the values the wide kernels produce, end to end, against the oracle."""
    w = synth.make_workload(name, B=B)
    got, want = run_both(oracle, w)
    compare(got, want)


@pytest.mark.parametrize("model,kw", CASES)
@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_schedule_built_on_the_device(oracle, model, kw, pairing):
    """schedule="device": the graph feed goes to the GPU, cavs_schedule_arena builds every index
    list there and the host only learns the round offsets.  Same results as with the host
    scheduler, against the oracle; the schedule read back from the device lists equals the
    oracle's trace; and several steps in a row alternate the two sets of list buffers."""
    loss = "softmax" if model != "treefc" else "root_sq"
    batches = [small_workload(model, 171 + k, B=5 + 4 * k, H=32, E=12, V=31, C=5) for k in range(3)]
    E = 32 if model == "lstm" else 12
    names = {"treelstm": ("Emb", "W", "U", "Bv"), "lstm": ("Emb", "W", "Bv"),
             "treefc": ("W", "Bv") if kw.get("use_bias") else ("W",)}[model]
    if loss == "softmax":
        names += ("Wfc", "bfc")
    s = session.Session(model, H=32, E=E, V=31, C_=5, pairing=pairing, loss=loss, schedule="device", **kw)
    s.set_params({k: batches[0]["params"][k] for k in names})
    for step, w in enumerate(batches + batches[:1]):
        print(f"[case] device schedule {model} {kw} pairing={pairing} step {step} N={w['N']}", flush=True)
        want = oracle.model_step(model, w["graph"], w["x"], w["labels"], batches[0]["params"], H=32, E=E, V=31, Cc=5,
                                 pairing=pairing, loss=loss, precise=True, **kw)
        s.step(w["graph"], w["x"], w["labels"], backward=True)
        got = dict(loss=s.fetch("loss"), graph_out=s.fetch("graph_out"), dgraph_out=s.fetch("dgraph_out"),
                   msg_pool=s.fetch("msg_pool"), grads=s.grads())
        got["trace"] = s.schedule_trace()
        assert got["trace"] == oracle.sched_trace(w["graph"])
        assert s.counter("scheduler") == 1, "the lists of this step were not built on the device"
        compare(got, want, loss=loss)
    s.close()


def test_device_scheduler_refuses_samples_it_cannot_hold():
    """Samples of more than 2048 vertices are the host scheduler's: the device scheduler says so
    instead of quietly handing the feed over."""
    T = 2100
    graph = np.full((1, T), -1, np.int32)
    graph[0, : T - 1] = np.arange(1, T)
    x, labels = np.zeros(T, np.float32), np.zeros(T, np.float32)
    s = session.Session("lstm", H=16, V=7, C_=3, schedule="device")
    with pytest.raises(hip.CavsError, match="at most 2048 vertices"):
        s.step(graph, x, labels, backward=False)
    s.close()
    s = session.Session("lstm", H=16, V=7, C_=3, schedule="host")
    s.step(graph, x, labels, backward=False)
    assert s.N == T and s.counter("scheduler") == 0
    s.close()


def test_device_schedule_rejects_what_the_host_scheduler_rejects():
    s = session.Session("treelstm", H=8, E=8, V=10, C_=3, schedule="device")
    with pytest.raises(hip.CavsError, match="terminator"):
        s.step(np.array([[1, 2, 0]], np.int32), np.zeros(3), np.zeros(3))
    with pytest.raises(hip.CavsError, match="single-vertex"):
        s.step(np.array([[-1, -1], [1, -1]], np.int32), np.zeros(3), np.zeros(3))
    with pytest.raises(hip.CavsError, match="out of range"):
        s.step(np.array([[7, 2, -1]], np.int32), np.zeros(3), np.zeros(3))
    with pytest.raises(hip.CavsError, match="cycle"):
        s.step(np.array([[1, 0, 3, -1]], np.int32), np.zeros(4), np.zeros(4))
    with pytest.raises(hip.CavsError, match="two children|mixes"):
        c = session.Session("lstm", H=8, V=10, C_=3, schedule="device")
        c.step(np.array([[2, 2, -1]], np.int32), np.zeros(3), np.zeros(3))
    s.close()


@pytest.mark.parametrize("schedule", ["host", "device"])
def test_plan_cache_replays_a_batch_structure_seen_before(oracle, schedule):
    """plan_cache=2: three structures cycled.  A structure met again within the last two skips the
    scheduler and the upload (plan_hits counts it) and gives the same step bit for bit as the
    first time; the third structure evicts the least recently used one.  New vertex inputs on a
    cached structure are a new computation on the old plan."""
    ws = [small_workload("treelstm", 181 + k, B=6 + k, H=32, E=12, V=31, C=5) for k in range(3)]
    s = session.Session("treelstm", H=32, E=12, V=31, C_=5, schedule=schedule, plan_cache=2)
    s.set_params(ws[0]["params"])
    seen = {}
    order = [0, 1, 0, 0, 2, 0, 1]        # hits at steps 2, 3, 5; step 4 evicts plan 1; step 6 misses again
    want_hits = [0, 0, 1, 2, 2, 3, 3]
    for step, k in enumerate(order):
        w = ws[k]
        print(f"[case] plan cache schedule={schedule} step {step} structure {k}", flush=True)
        s.step(w["graph"], w["x"], w["labels"], backward=True)
        got = (s.fetch("loss"), s.fetch("graph_out"), s.grads())
        assert s.counter("plan_hits") == want_hits[step], (step, s.counter("plan_hits"))
        assert s.schedule_trace() == oracle.sched_trace(w["graph"])
        if k in seen:
            np.testing.assert_array_equal(got[0], seen[k][0])
            np.testing.assert_array_equal(got[1], seen[k][1])
            for name in ("dW", "dU", "dBv", "dWfc"):
                np.testing.assert_array_equal(got[2][name], seen[k][2][name])
        else:
            want = oracle.model_step("treelstm", w["graph"], w["x"], w["labels"], ws[0]["params"], H=32, E=12, V=31, Cc=5,
                                     precise=True)
            close(got[0], want["loss"], "loss")
            close(got[2]["dU"], want["grads"]["dU"], "dU")
            seen[k] = got
    # the same structure with other words: a hit, and the oracle's result for the new inputs
    w = ws[0]
    x2 = ((w["x"] + 3) % 31).astype(np.float32)
    s.step(w["graph"], x2, w["labels"], backward=True)
    assert s.counter("plan_hits") == 4
    want = oracle.model_step("treelstm", w["graph"], x2, w["labels"], ws[0]["params"], H=32, E=12, V=31, Cc=5, precise=True)
    close(s.fetch("loss"), want["loss"], "loss with new inputs")
    close(s.grads()["dW"], want["grads"]["dW"], "dW with new inputs")
    s.close()


def test_steps_are_repeatable_and_sessions_reusable(oracle):
    """Two different batches through one session (buffers grow, lists are re-uploaded),
    then the first again: identical results, no state leaks between steps."""
    a = small_workload("treelstm", 71, B=4, H=16, E=12)
    b = small_workload("treelstm", 72, B=9, H=16, E=12)
    s = session.Session("treelstm", H=16, E=12, V=a["V"], C_=a["C"])
    s.set_params(a["params"])
    outs = []
    for w in (a, b, a):
        print(f"[case] reuse N={w['N']}", flush=True)
        s.step(w["graph"], w["x"], w["labels"])
        outs.append((s.fetch("loss"), s.grads()))
    np.testing.assert_array_equal(outs[0][0], outs[2][0])
    for k in ("dW", "dU", "dBv", "dWfc"):
        np.testing.assert_array_equal(outs[0][1][k], outs[2][1][k])
    want = oracle.model_step("treelstm", b["graph"], b["x"], b["labels"], a["params"], H=16, E=12, V=a["V"], Cc=a["C"],
                             precise=True)
    close(outs[1][0], want["loss"], "loss of second batch")
    s.close()


def test_device_resident_feeds_and_sgd(oracle):
    import torch

    w = small_workload("lstm", 73, B=5, H=16)
    s = session.Session("lstm", H=16, V=w["V"], C_=w["C"])
    s.set_params(w["params"])
    x = torch.from_numpy(w["x"]).cuda()
    lab = torch.from_numpy(w["labels"]).cuda()
    torch.cuda.synchronize()
    s.step(w["graph"], x, lab, backward=True, lr=0.5)
    g = s.grads()
    want = oracle.model_step("lstm", w["graph"], w["x"], w["labels"], w["params"], H=16, V=w["V"], Cc=w["C"], precise=True)
    close(g["dW"], want["grads"]["dW"], "dW")
    close(s.param("W", (8 * 16 * 16,)), w["params"]["W"] - np.float32(0.5) * g["dW"], "W after SGD", rtol=1e-6, atol=1e-7)
    assert s.timing("RNNForward") > 0 and s.timing("RNNBackward") > 0 and s.timing("GraphParsing") >= 0
    assert s.counter("gemm_flops") > 0 and s.counter("rounds") == len(oracle.sched_trace(w["graph"])["fwd"])
    s.close()


def test_error_paths_do_not_touch_the_device():
    s = session.Session("treelstm", H=8, E=8, V=10, C_=3)
    with pytest.raises(hip.CavsError, match="no parameter named"):
        s.set_params({"nope": np.zeros(3)})
    with pytest.raises(hip.CavsError, match="elements"):
        s.set_params({"W": np.zeros(3)})
    with pytest.raises(hip.CavsError, match="terminator"):
        s.step(np.array([[1, 2, 0]], np.int32), np.zeros(3), np.zeros(3))
    with pytest.raises(hip.CavsError, match="single-vertex"):
        s.step(np.array([[-1, -1], [1, -1]], np.int32), np.zeros(3), np.zeros(3))
    with pytest.raises(hip.CavsError, match="two children|mixes"):
        c = session.Session("lstm", H=8, V=10, C_=3)
        c.step(np.array([[2, 2, -1]], np.int32), np.zeros(3), np.zeros(3))
    s.close()


# ---- full-size properties (no oracle: too slow on one core) ----
def test_full_size_tree_lstm_properties():
    """C3 at full size: permuting the samples of a batch permutes nothing but rows
    (row-id pairing), gradients are finite, and the loss equals the fp64 cross-entropy
    of the returned hidden states."""
    w = synth.make_workload("C3")
    p = w["params"]
    s = session.Session("treelstm", H=w["H"], E=w["E"], V=w["V"], C_=w["C"], pairing="rowid")
    s.set_params(p)
    print(f"[case] C3 full N={w['N']}", flush=True)
    s.step(w["graph"], w["x"], w["labels"])
    GO, loss, g = s.fetch("graph_out"), s.fetch("loss"), s.grads()
    logits = GO.astype(np.float64) @ p["Wfc"].astype(np.float64).T + p["bfc"]
    lse = np.log(np.exp(logits - logits.max(1, keepdims=True)).sum(1)) + logits.max(1)
    close(loss, lse - logits[np.arange(w["N"]), w["labels"].astype(int)], "loss vs fp64 head")
    assert all(np.isfinite(v).all() for v in g.values())
    assert np.abs(g["dW"]).max() > 0 and np.abs(g["dU"]).max() > 0
    # reverse the sample order
    lens = [int(np.argmax(r == -1)) + 1 for r in w["graph"]]
    offs = np.concatenate([[0], np.cumsum(lens)])
    order = list(range(w["B"]))[::-1]
    g2 = w["graph"][order]
    idx = np.concatenate([np.arange(offs[i], offs[i + 1]) for i in order])
    s.step(g2, w["x"][idx], w["labels"][idx])
    close(s.fetch("graph_out"), GO[idx], "graph_out under sample permutation", rtol=1e-5, atol=1e-6)
    gp = s.grads()
    for k in ("dW", "dU", "dBv", "dWfc", "dbfc"):
        close(gp[k], g[k], k + " under sample permutation")
    s.close()


@pytest.mark.parametrize("name", ["C3", "C4", "C5"])
def test_full_size_fused_rounds_equal_separate_launches(name):
    """At the benchmark's own sizes the two ways a round runs -- one fused launch, or gather,
    GEMMs, gates and scatter as separate launches -- must give the same step (they share no
    MFMA kernel: the fused rounds feed the matrix cores from global memory, the separate path
    goes through the LDS-tiled GEMM; the deferred products are grouped in both)."""
    w = synth.make_workload(name)
    kw = dict(H=w["H"], E=w["E"], V=w["V"], C_=w["C"])
    outs = []
    for limit in (0, -1):
        print(f"[case] {name} full N={w['N']} fused_round_rows={limit}", flush=True)
        s = session.Session(w["model"], fused_round_rows=limit, **kw)
        s.set_params(w["params"])
        s.step(w["graph"], w["x"], w["labels"], backward=True)
        outs.append(dict(loss=s.fetch("loss"), go=s.fetch("graph_out"), grads=s.grads(), rf=s.counter("round_flops")))
        s.close()
    assert outs[0]["rf"] > 0 and outs[1]["rf"] == 0  # the first really ran fused rounds, the second none
    close(outs[0]["loss"], outs[1]["loss"], "loss")
    close(outs[0]["go"], outs[1]["go"], "graph_out")
    for k, v in outs[1]["grads"].items():
        close(outs[0]["grads"][k], v, k)


@pytest.mark.parametrize("H,limit", [(32, 0), (64, 0), (96, 0), (64, 20), (64, -1), (256, 0), (512, 0)])
@pytest.mark.parametrize("pairing", ["reference", "rowid"])
@pytest.mark.parametrize("model,kw", CASES)
def test_fused_rounds_match_oracle(oracle, model, kw, H, limit, pairing):
    """Whole rounds as single launches for all three vertex functions: 70 samples give rounds
    above 64 rows (32x32 tiles, or 16x16 with four wavefronts), between 17 and 64 (16x16 tiles)
    and down to one row.  limit=20 mixes fused and separate rounds in one step, -1 never fuses."""
    w = small_workload(model, 91, B=70, H=H, E=12, V=31, C=5)
    if model == "treefc" and H >= 256:
        # small_workload draws W from U(-0.4, 0.4) whatever H is.  A sum of 2H = 1024 such terms has a
        # standard deviation of 7: each level of the tree multiplies a rounding error of its inputs by
        # about that, and after ten levels no fp32 summation order is within 1e-5 of the exact value.
        # Scaled to the spread the benchmark's own U(-0.1, 0.1) has at H = 256.
        w["params"]["W"] = (w["params"]["W"] * np.float32(0.25 * np.sqrt(256.0 / H))).astype(np.float32)
    E = H if model == "lstm" else 12
    loss = "softmax" if model != "treefc" else "root_sq"
    print(f"[case] fused rounds {model} {kw} H={H} limit={limit} pairing={pairing} N={w['N']}", flush=True)
    want = oracle.model_step(model, w["graph"], w["x"], w["labels"], w["params"], H=H, E=E, V=31, Cc=5, pairing=pairing,
                             loss=loss, precise=True, threads=16, **kw)
    s = session.Session(model, H=H, E=E, V=31, C_=5, pairing=pairing, fused_round_rows=limit, loss=loss, **kw)
    names = {"treelstm": ("Emb", "W", "U", "Bv"), "lstm": ("Emb", "W", "Bv"),
             "treefc": ("W", "Bv") if kw.get("use_bias") else ("W",)}[model]
    if loss == "softmax":
        names += ("Wfc", "bfc")
    s.set_params({k: w["params"][k] for k in names})
    s.step(w["graph"], w["x"], w["labels"], backward=True)
    got = dict(loss=s.fetch("loss"), graph_out=s.fetch("graph_out"), dgraph_out=s.fetch("dgraph_out"),
               msg_pool=s.fetch("msg_pool"), grads=s.grads(), trace=s.schedule_trace())
    fused_flops = s.counter("round_flops")
    s.close()
    compare(got, want, loss=loss)
    assert (fused_flops > 0) == (limit >= 0), fused_flops


@pytest.mark.parametrize("pairing", ["reference", "rowid"])
@pytest.mark.parametrize("model,kw", CASES)
def test_backward_rounds_as_one_launch_or_two(oracle, model, kw, pairing):
    """A backward round either as two launches (gate gradients, then the children's d h through
    the pool) or as one that goes on to the children's gate gradients: both against the oracle,
    and the launch count shows that each really ran."""
    H = 64
    E = H if model == "lstm" else 12
    loss = "softmax" if model != "treefc" else "root_sq"
    w = small_workload(model, 57, B=40, H=H, E=12, V=31, C=5)
    want = oracle.model_step(model, w["graph"], w["x"], w["labels"], w["params"], H=H, E=E, V=31, Cc=5, pairing=pairing, loss=loss,
                             precise=True, threads=16, **kw)
    names = {"treelstm": ("Emb", "W", "U", "Bv"), "lstm": ("Emb", "W", "Bv"),
             "treefc": ("W", "Bv") if kw.get("use_bias") else ("W",)}[model]
    if loss == "softmax":
        names += ("Wfc", "bfc")
    launches = []
    for split in (False, True):
        print(f"[case] {model} {kw} backward rounds split={split} pairing={pairing} N={w['N']}", flush=True)
        s = session.Session(model, H=H, E=E, V=31, C_=5, pairing=pairing, split_backward_rounds=split, loss=loss, **kw)
        s.set_params({k: w["params"][k] for k in names})
        s.step(w["graph"], w["x"], w["labels"], backward=True)
        got = dict(loss=s.fetch("loss"), graph_out=s.fetch("graph_out"), dgraph_out=s.fetch("dgraph_out"),
                   msg_pool=s.fetch("msg_pool"), grads=s.grads(), trace=s.schedule_trace())
        launches.append(s.counter("launches"))
        s.close()
        compare(got, want, loss=loss)
    assert launches[0] < launches[1], launches


@pytest.mark.parametrize("name", ["C1", "C2", "C3"])
def test_a_step_is_reproducible_bit_for_bit(name):
    """Every sum on the path runs in a fixed order (partial tiles through LDS in wavefront order,
    split-K partials and column sums by index), so two runs of the same step agree bit for bit --
    all but the embedding gradient, whose repeated rows are added with atomics."""
    w = synth.make_workload(name)
    kw = dict(H=w["H"], E=w["E"], V=w["V"], C_=w["C"])
    if w["model"] == "treefc":
        kw.update(loss="root_sq", act=1, use_bias=True, use_x=True)
    runs = []
    for k in range(2):
        print(f"[case] {name} reproducibility run {k}", flush=True)
        s = session.Session(w["model"], **kw)
        s.set_params(w["params"])
        s.step(w["graph"], w["x"], w["labels"], backward=True)
        runs.append(dict(loss=s.fetch("loss"), go=s.fetch("graph_out"), dgo=s.fetch("dgraph_out"), grads=s.grads()))
        s.close()
    for k in ("loss", "go", "dgo"):
        np.testing.assert_array_equal(runs[0][k], runs[1][k], err_msg=k)
    for k, v in runs[0]["grads"].items():
        if k == "dEmb":
            close(v, runs[1]["grads"][k], k)
        else:
            np.testing.assert_array_equal(v, runs[1]["grads"][k], err_msg=k)


@pytest.mark.parametrize("model", ["treelstm", "lstm"])
def test_training_steps_with_the_row_sparse_embedding_update(oracle, model):
    """Four SGD steps over three different batches (token ids overlap between steps, one
    step runs without an update in between): every parameter, the embedding table in
    particular, follows the oracle's dense w -= lr * g, and the gradients of the last step
    stay readable."""
    kw = dict(B=6, H=32, E=12, V=17, C=4)            # a tiny vocabulary: many repeated rows
    batches = [small_workload(model, 101 + k, **kw) for k in range(3)]
    H, E, V, C_ = 32, (32 if model == "lstm" else 12), 17, 4
    s = session.Session(model, H=H, E=E, V=V, C_=C_)
    s.set_params(batches[0]["params"])
    names = ("Emb", "W", "U", "Bv", "Wfc", "bfc") if model == "treelstm" else ("Emb", "W", "Bv", "Wfc", "bfc")
    p = {k: np.array(batches[0]["params"][k], np.float32) for k in names}
    plan = [(0, 0.5), (1, 0.0), (2, 0.25), (0, 0.5)]  # (batch, lr); lr 0 leaves the gradient in place
    for step, (bi, lr) in enumerate(plan):
        w = batches[bi]
        print(f"[case] {model} sgd step {step} batch {bi} lr {lr}", flush=True)
        want = oracle.model_step(model, w["graph"], w["x"], w["labels"], p, H=H, E=E, V=V, Cc=C_, precise=True, threads=16)
        s.step(w["graph"], w["x"], w["labels"], backward=True, lr=lr)
        got = s.grads()
        for k in names:
            close(got["d" + k], want["grads"]["d" + k], f"d{k} at step {step}")
            p[k] = (p[k] - np.float32(lr) * want["grads"]["d" + k].reshape(p[k].shape)).astype(np.float32)
    for k in names:
        close(s.param(k, p[k].shape), p[k], f"{k} after the steps")
    s.close()


@pytest.mark.parametrize("model,H", [("treelstm", 128), ("lstm", 256)])
def test_the_packed_copy_of_the_recurrent_weights_follows_every_writer(oracle, model, H):
    """Rounds of more than 64 vertices at these hidden sizes read the recurrent weights (U; W' of
    the chain LSTM) from their tile-major copy.  The copy is written by the update job; set_param
    writes the weights behind its back.  Three steps -- the first packs on demand, the second reads
    what the first step's update left, the third follows a set_params -- each against the oracle
    on the parameters the session should hold."""
    E, V, C_ = (16 if model == "treelstm" else H), 37, 5
    w = small_workload(model, 333, B=70, H=H, E=E, V=V, C=C_, skew=False)
    rec = "U" if model == "treelstm" else "W"
    names = ("Emb", "W", "U", "Bv", "Wfc", "bfc") if model == "treelstm" else ("Emb", "W", "Bv", "Wfc", "bfc")
    p = {k: np.array(w["params"][k], np.float32) for k in names}
    p[rec] = (p[rec] * np.float32(0.2)).astype(np.float32)
    s = session.Session(model, H=H, E=E, V=V, C_=C_)
    ok = hip.lib().cavs_round_packed_ok if model == "treelstm" else hip.lib().cavs_lstm_round_packed_ok
    assert ok(70, H) == 1
    s.set_params(p)
    lr = 0.25
    for step in range(3):
        print(f"[case] packed copy {model} step {step}", flush=True)
        if step == 2:
            p[rec] = (p[rec][::-1] * np.float32(0.5)).astype(np.float32)
            s.set_params({rec: p[rec]})
        want = oracle.model_step(model, w["graph"], w["x"], w["labels"], p, H=H, E=E, V=V, Cc=C_, precise=True, threads=16)
        s.step(w["graph"], w["x"], w["labels"], backward=True, lr=lr)
        close(s.fetch("graph_out"), want["graph_out"], f"graph_out at step {step}")
        got = s.grads()
        for k in names:
            close(got["d" + k], want["grads"]["d" + k], f"d{k} at step {step}")
            p[k] = (p[k] - np.float32(lr) * want["grads"]["d" + k].reshape(p[k].shape)).astype(np.float32)
    close(s.param(rec, p[rec].shape), p[rec], f"{rec} after the steps")
    s.close()


def test_the_transposed_copy_of_a_wide_heads_weights_follows_every_writer(oracle):
    """A classifier of C * H >= 2^18 weights is multiplied through an [H, C] copy of them.  The copy is
    written by the update job; set_param writes the weights behind its back.  Three steps -- the
    first copies on demand, the second reads what the first step's update left, the third follows
    a set_params -- each against the oracle on the parameters the session should hold."""
    model, H, V, C_ = "lstm", 64, 37, 4100
    w = small_workload(model, 77, B=6, H=H, E=H, V=V, C=C_, skew=False)
    names = ("Emb", "W", "Bv", "Wfc", "bfc")
    p = {k: np.array(w["params"][k], np.float32) for k in names}
    s = session.Session(model, H=H, E=H, V=V, C_=C_)
    s.set_params(p)
    lr = 0.25
    for step in range(3):
        print(f"[case] wide head step {step}", flush=True)
        if step == 2:
            p["Wfc"] = (p["Wfc"][::-1] * np.float32(0.5)).astype(np.float32)
            s.set_params({"Wfc": p["Wfc"]})
        want = oracle.model_step(model, w["graph"], w["x"], w["labels"], p, H=H, E=H, V=V, Cc=C_, precise=True, threads=16)
        s.step(w["graph"], w["x"], w["labels"], backward=True, lr=lr)
        close(s.fetch("loss"), want["loss"], f"loss at step {step}")
        close(s.fetch("dgraph_out"), want["dgraph_out"], f"dgraph_out at step {step}")
        got = s.grads()
        for k in names:
            close(got["d" + k], want["grads"]["d" + k], f"d{k} at step {step}")
            p[k] = (p[k] - np.float32(lr) * want["grads"]["d" + k].reshape(p[k].shape)).astype(np.float32)
    close(s.param("Wfc", p["Wfc"].shape), p["Wfc"], "Wfc after the steps")
    s.close()


@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_a_wide_head_in_chunks_beside_the_rounds(oracle, pairing):
    """Chain LSTM with a wide classifier: the head runs on a second stream over chunks of the rounds,
    last chunk first, while the backward rounds of the chunks already done run.  Sequences of 4..30
    steps end in every chunk (the vertices nobody sends a gradient to are handled chunk by chunk).
    Six training steps on changing batches (two of them met before, the last one larger than the
    buffers) against the oracle: two chunks
    (the default), four, two with a plan cache (the chunks of a structure met again come out of the
    cache), and the head in one piece."""
    model, H, V, C_ = "lstm", 64, 41, 4096
    rng = synth.SplitMix64(91)
    p = dict(Emb=rng.bulk_normal(V * H, 0, 0.5).reshape(V, H), W=rng.bulk_uniform(8 * H * H, -0.3, 0.3), Bv=rng.bulk_uniform(4 * H, -0.3, 0.3),
             Wfc=rng.bulk_uniform(C_ * H, -0.3, 0.3).reshape(C_, H), bfc=rng.bulk_uniform(C_, -0.2, 0.2))
    p = {k: np.asarray(v, np.float32) for k, v in p.items()}
    lr = 0.2
    sessions = {hc: session.Session(model, H=H, E=H, V=V, C_=C_, pairing=pairing, head_chunks=hc) for hc in (0, 4, -1)}
    sessions["cache"] = session.Session(model, H=H, E=H, V=V, C_=C_, pairing=pairing, plan_cache=4)
    for s in sessions.values():
        s.set_params(p)
    for step, seed in enumerate([500, 501, 500, 502, 501, 503]):
        # (the last batch is half as large again: every per-vertex buffer is reallocated)
        graph, lens, _ = synth.chain_batch(seed, 40, 22 if seed == 503 else 4, 30, 30)
        N = sum(lens)
        x = np.floor(rng.bulk_uniform(N) * V).astype(np.float32)
        labels = np.floor(rng.bulk_uniform(N) * C_).astype(np.float32)
        want = oracle.model_step(model, graph, x, labels, p, H=H, E=H, V=V, Cc=C_, pairing=pairing, precise=True, threads=16)
        for hc, s in sessions.items():
            print(f"[case] wide head, head_chunks={hc}, step {step}, N={N}, pairing={pairing}", flush=True)
            s.step(graph, x, labels, backward=True, lr=lr)
            assert s.counter("head_chunks") == {0: 2, 4: 4, -1: 0, "cache": 2}[hc]
            for k in ("loss", "graph_out", "dgraph_out"):
                close(s.fetch(k), want[k], f"{k} at step {step}", scaled=False)
            got = s.grads()
            for k in p:
                close(got["d" + k], want["grads"]["d" + k], f"d{k} at step {step}", scaled=False)
        for k in p:
            p[k] = (p[k] - np.float32(lr) * want["grads"]["d" + k].reshape(p[k].shape)).astype(np.float32)
    assert sessions["cache"].counter("plan_hits") == 2
    for s in sessions.values():
        close(s.param("Wfc", p["Wfc"].shape), p["Wfc"], "Wfc after the steps")
        close(s.param("W", p["W"].shape), p["W"], "W after the steps")
        s.close()


@pytest.mark.parametrize("kind", ["trees", "tokens"])
def test_training_step_on_reader_batches(oracle, kind):
    """The text readers (cavs_amd/data.py) feed the session directly: the fixture corpora
    through one training step, against the oracle on the same arrays."""
    import os

    from cavs_amd import data

    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    if kind == "trees":
        r = data.TreeReader(*[os.path.join(golden, "sst_tiny", f) for f in ("sents_idx.txt", "labels.txt", "parents.txt")],
                            batch=3, max_vertices=9, max_words=5)
        graph, x, labels = r.next_batch(pack_inputs=True)
        model, V, C = "treelstm", 21, 5
    else:
        r = data.PtbReader(os.path.join(golden, "ptb_tiny.txt"), batch=2, max_length=5)
        graph, x, labels = r.batch_at(2)
        model, V, C = "lstm", 23, 23
    N = sum(int(np.argmax(row == -1)) + 1 for row in graph)  # a sample ends at its first -1, the root
    x, labels = x[:N].copy(), labels[:N].copy()
    labels[labels < 0] = 0  # the last token of a sentence has no successor: class 0
    w = small_workload(model, 77, H=16, E=16, V=V, C=C)
    w.update(graph=graph, x=x, labels=labels, N=N)
    print(f"[case] reader kind={kind} N={N}", flush=True)
    got, want = run_both(oracle, w)
    compare(got, want)


@pytest.mark.parametrize("model,H,pool,Cc", [("treefc", 32, 3, 5), ("treelstm", 32, 3, 5), ("lstm", 32, 2, 5), ("treelstm", 512, 2, 5),
                                             ("lstm", 32, 2, 9000)])
def test_recorded_graph_of_a_cached_plan_gives_the_steps_of_the_host_loop(model, H, pool, Cc):
    """graph_replay: on a batch structure seen before, with the same device-resident feeds, the
    forward pass, loss head and backward pass are enqueued as one recorded graph.  Training steps
    (with the parameter update) through such a session and through one that issues every launch
    from the host loop give the same losses and parameters -- bit for bit where no gradient is
    accumulated with atomics (Tree-FC), to the tolerance of the accumulation order elsewhere.
    H = 512 puts the launches over the rounds near the roots inside the graph; 9000 classes make the
    head a wide one (its weight gradient goes to a side stream in the session that does not record)."""
    import torch
    V = 31
    E = H if model == "lstm" else 12
    loss = "softmax" if model != "treefc" else "root_sq"
    ws = [small_workload(model, 401 + k, B=5 + k, H=H, E=E, V=V, C=Cc) for k in range(pool)]
    names = {"treelstm": ("Emb", "W", "U", "Bv", "Wfc", "bfc"), "lstm": ("Emb", "W", "Bv", "Wfc", "bfc"), "treefc": ("W",)}[model]
    params = {k: np.asarray(ws[0]["params"][k], np.float32) for k in names}
    sessions = [session.Session(model, H=H, E=E, V=V, C_=Cc, loss=loss, plan_cache=4, graph_replay=bool(r)) for r in (0, 1)]
    for s in sessions:
        s.set_params(params)
    feeds = [(w["graph"], torch.from_numpy(np.ascontiguousarray(w["x"], np.float32)).cuda(),
              torch.from_numpy(np.ascontiguousarray(w["labels"], np.float32)).cuda()) for w in ws]
    torch.cuda.synchronize()
    steps = 5 * pool
    for i in range(steps):
        g, x, lab = feeds[i % pool]
        print(f"[case] graph replay {model} H={H} step {i}", flush=True)
        losses = []
        for s in sessions:
            s.step(g, x, lab, backward=True, lr=0.05)
            losses.append(s.fetch("loss"))
        if model == "treefc":
            np.testing.assert_array_equal(losses[1], losses[0])
        else:
            np.testing.assert_allclose(losses[1], losses[0], rtol=2e-5, atol=1e-6)
    assert sessions[0].counter("graph_replays") == 0
    # every structure: a miss, then a recording, then replays (an odd cycle of structures meets each
    # of the two id buffers in turn and records once per buffer)
    assert sessions[1].counter("graph_replays") >= steps - 2 * pool, sessions[1].counter("graph_replays")
    assert sessions[1].counter("plan_hits") == steps - pool
    for n in names:
        a, b = (s.param(n, params[n].shape) for s in sessions)
        if model == "treefc":
            np.testing.assert_array_equal(b, a)
        else:
            np.testing.assert_allclose(b, a, rtol=2e-5, atol=2e-6)
    # a call in between (new parameters) makes the next step an ordinary one, with the host loop's result
    for s in sessions:
        s.set_params(params)
    g, x, lab = feeds[0]
    out = []
    for s in sessions:
        s.step(g, x, lab, backward=True, lr=0.0)
        out.append(s.fetch("loss"))
    np.testing.assert_allclose(out[1], out[0], rtol=2e-6, atol=1e-7)
    for s in sessions:
        s.close()
