"""Pins oracle/model.c + oracle/ops.c gate math against independent fp64
formulations (tests/textbook.py)."""
import numpy as np
import pytest

import textbook
from cavs_amd import synth

RTOL, ATOL = 1e-4, 1e-5  # the fp32 bar of the path; the oracle itself is fp32


def _close(a, b, what, rtol=RTOL, atol=ATOL):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    assert a.shape == b.shape, what
    err = np.abs(a - b)
    # scale the absolute floor by the tensor's magnitude so tiny gradients are judged fairly
    tol = atol * max(1.0, float(np.abs(b).max())) + rtol * np.abs(b)
    bad = err > tol
    assert not bad.any(), f"{what}: max err {err.max():.3e} at {int(err.argmax())} (ref {b[err.argmax()]:.3e})"


def small_workload(model, seed, B=5, H=12, E=10, V=37, C=5, skew=True):
    rng = synth.SplitMix64(seed)
    if model == "lstm":
        graph, lens, _ = synth.chain_batch(seed, B, 2 if skew else 6, 9 if skew else 6, 9)
        N = sum(lens)
        E = H
    else:
        if skew:
            graph, leaves, _ = synth.tree_batch(seed, B, 2, 8, 15)
        else:  # one bracketing replicated: every round holds the same vertex of every sample
            tree = synth.random_binary_tree(synth.SplitMix64(seed + 1), 6)
            graph, leaves = synth.pack_graph([tree] * B, 15), [6] * B
        N = sum(2 * l - 1 for l in leaves)
    p = {}
    if model in ("treelstm", "treelstm2"):  # (treelstm2: a forget-gate matrix per child, U = [U_iou | U_fl | U_fr])
        p = dict(Emb=rng.bulk_normal(V * E, 0, 0.5).reshape(V, E),
                 W=rng.bulk_uniform(E * 4 * H, -0.4, 0.4).reshape(E, 4 * H),
                 U=rng.bulk_uniform((5 if model == "treelstm2" else 4) * H * H, -0.4, 0.4), Bv=rng.bulk_uniform(4 * H, -0.3, 0.3))
        x = np.floor(rng.bulk_uniform(N) * V).astype(np.float32)
    elif model == "treegate":  # (textbook._treegate_cell: one state block, no oracle restatement)
        p = dict(Emb=rng.bulk_normal(V * E, 0, 0.5).reshape(V, E), W=rng.bulk_uniform(E * 2 * H, -0.4, 0.4),
                 U=rng.bulk_uniform(3 * H * H, -0.3, 0.3), Bv=rng.bulk_uniform(2 * H, -0.3, 0.3))
        x = np.floor(rng.bulk_uniform(N) * V).astype(np.float32)
    elif model in ("treegru", "treedeep"):  # (textbook._treegru_cell, _treedeep_cell: two and three stages of products, no oracle restatement)
        g = 3 if model == "treegru" else 2
        p = dict(Emb=rng.bulk_normal(V * E, 0, 0.5).reshape(V, E), W=rng.bulk_uniform(E * g * H, -0.4, 0.4),
                 U=rng.bulk_uniform(g * H * H, -0.3, 0.3), Bv=rng.bulk_uniform(g * H, -0.3, 0.3))
        x = np.floor(rng.bulk_uniform(N) * V).astype(np.float32)
    elif model == "lstm":
        p = dict(Emb=rng.bulk_normal(V * H, 0, 0.5).reshape(V, H),
                 W=rng.bulk_uniform(8 * H * H, -0.4, 0.4), Bv=rng.bulk_uniform(4 * H, -0.3, 0.3))
        x = np.floor(rng.bulk_uniform(N) * V).astype(np.float32)
    else:
        p = dict(W=rng.bulk_uniform(2 * H * H, -0.4, 0.4).reshape(2 * H, H),
                 Bv=rng.bulk_uniform(H, -0.3, 0.3))
        x = rng.bulk_normal(N * H).reshape(N, H)
    p["Wfc"] = rng.bulk_uniform(C * H, -0.5, 0.5).reshape(C, H)
    p["bfc"] = rng.bulk_uniform(C, -0.2, 0.2)
    labels = np.floor(rng.bulk_uniform(N) * C).astype(np.float32)
    return dict(model=model, graph=graph, x=x, labels=labels, params=p, H=H, E=E, V=V, C=C, N=N)


def _run_oracle(oracle, w, **kw):
    return oracle.model_step(w["model"], w["graph"], w["x"], w["labels"], w["params"], H=w["H"],
                             E=w["E"], V=w["V"], Cc=w["C"], **kw)


def _compare(res, ref, grads=True):
    _close(res["loss"], ref["loss"], "loss")
    _close(res["graph_out"], ref["graph_out"], "graph_out")
    _close(res["dgraph_out"], ref["dgraph_out"], "dgraph_out")
    if grads:
        for k, v in res["grads"].items():
            if k in ref["grads"]:
                _close(v, ref["grads"][k], k)


CASES = [("treelstm", dict()), ("lstm", dict()), ("treefc", dict(act=1, use_bias=True, use_x=True)),
         ("treefc", dict(act=0)), ("treelstm2", dict())]


@pytest.mark.parametrize("model,kw", CASES)
@pytest.mark.parametrize("loss", ["softmax", "root_sq"])
@pytest.mark.parametrize("seed", [11, 12])
def test_rowid_pairing_equals_textbook_per_sample(oracle, model, kw, loss, seed):
    w = small_workload(model, seed)
    ref = textbook.per_sample(model, w["graph"], w["x"], w["labels"], w["params"], w["H"], loss=loss, **kw)
    res = _run_oracle(oracle, w, loss=loss, pairing="rowid", **kw)
    _compare(res, ref)


@pytest.mark.parametrize("model,kw", CASES)
def test_serial_scheduler_equals_textbook_per_sample(oracle, model, kw):
    """SerialGraphScheduler (no OPT_BATCHING) is unaffected by the pairing."""
    w = small_workload(model, 21)
    ref = textbook.per_sample(model, w["graph"], w["x"], w["labels"], w["params"], w["H"], **kw)
    for pairing in ("reference", "rowid"):
        res = _run_oracle(oracle, w, batching=False, pairing=pairing, **kw)
        _compare(res, ref)


@pytest.mark.parametrize("model,kw", CASES)
def test_reference_pairing_on_same_shape_batch_equals_textbook(oracle, model, kw):
    w = small_workload(model, 31, skew=False)
    ref = textbook.per_sample(model, w["graph"], w["x"], w["labels"], w["params"], w["H"], **kw)
    res = _run_oracle(oracle, w, pairing="reference", **kw)
    _compare(res, ref)


@pytest.mark.parametrize("model,kw", CASES)
@pytest.mark.parametrize("loss", ["softmax", "root_sq"])
@pytest.mark.parametrize("seed", [41, 42, 43])
def test_reference_pairing_backward_is_transpose_of_forward(oracle, model, kw, loss, seed):
    """Skewed batch, the reference's b-th-entry pairing: autograd of the same
    dataflow must equal the hand-written backward."""
    w = small_workload(model, seed)
    tr = oracle.sched_trace(w["graph"])
    ref = textbook.round_based(model, w["graph"], tr, w["x"], w["labels"], w["params"], w["H"],
                               loss=loss, pairing="reference", **kw)
    res = _run_oracle(oracle, w, loss=loss, pairing="reference", **kw)
    _compare(res, ref)


def test_reference_pairing_differs_from_textbook_on_skewed_batch(oracle):
    """The shifted rows are real: on the hand-derived two-tree batch the reference
    pairing hands sample 0's root state to sample 1's root."""
    graph = np.array([[2, 2, -1, -1, -1], [3, 3, 4, 4, -1]], np.int32)
    w = small_workload("treefc", 5)
    H = w["H"]
    x = synth.SplitMix64(9).bulk_normal(8 * H).reshape(8, H)
    kw = dict(act=1, use_bias=True, use_x=True, loss="sum_abs")
    ref = oracle.model_step("treefc", graph, x, np.zeros(8), w["params"], H=H, pairing="rowid", **kw)
    quirk = oracle.model_step("treefc", graph, x, np.zeros(8), w["params"], H=H, pairing="reference", **kw)
    # pool row 6 (vertex 6's message) holds vertex 2's state under the reference pairing
    np.testing.assert_array_equal(quirk["msg_pool"][6], quirk["graph_out"][2])
    np.testing.assert_array_equal(ref["msg_pool"][6], ref["graph_out"][6])
    assert not np.allclose(ref["graph_out"][7], quirk["graph_out"][7])
    # everything not downstream of the shifted row is untouched
    np.testing.assert_array_equal(ref["graph_out"][:7], quirk["graph_out"][:7])


def test_swapping_samples_makes_reference_pairing_correct(oracle):
    graph = np.array([[3, 3, 4, 4, -1], [2, 2, -1, -1, -1]], np.int32)
    w = small_workload("treelstm", 6)
    N = 8
    x, labels = w["x"][:N], w["labels"][:N]
    ref = textbook.per_sample("treelstm", graph, x, labels, w["params"], w["H"])
    res = oracle.model_step("treelstm", graph, x, labels, w["params"], H=w["H"], E=w["E"], V=w["V"],
                            Cc=w["C"], pairing="reference")
    _compare(res, ref)


def test_sum_abs_loss_has_the_gradient_of_a_plain_sum(oracle):
    """Reduce_sum is cublasSasum (sum of |x|) but its gradient op is a constant
    fill (op_impl_blas1_cublas.cc:62-77, op_decl_reduction.cc:19-28)."""
    w = small_workload("treelstm", 51)
    res = _run_oracle(oracle, w, loss="sum_abs", pairing="rowid")
    assert (res["graph_out"] < 0).any()
    _close(res["loss"], [np.abs(res["graph_out"].astype(np.float64)).sum()], "sum|h|")
    np.testing.assert_array_equal(res["dgraph_out"], np.ones_like(res["dgraph_out"]))


# ---- the double-precision build of the same sources (ord_*): what the fp32 GPU results are
# held to the path's tolerance against.  It must (a) be the same dataflow as the fp32 build and
# (b) really hold every value and sum in double -- a single float intermediate would leave an
# error of ~1e-7 relative, far above the 1e-11 asked for here.
TIGHT = dict(rtol=1e-10, atol=1e-12)


def _compare_tight(res, ref):
    assert res["loss"].dtype == np.float64
    _close(res["loss"], ref["loss"], "loss", **TIGHT)
    _close(res["graph_out"], ref["graph_out"], "graph_out", **TIGHT)
    _close(res["dgraph_out"], ref["dgraph_out"], "dgraph_out", **TIGHT)
    for k, v in res["grads"].items():
        if k in ref["grads"]:
            _close(v, ref["grads"][k], k, **TIGHT)


@pytest.mark.parametrize("model,kw", CASES)
@pytest.mark.parametrize("loss", ["softmax", "root_sq"])
def test_double_build_equals_fp64_textbook_to_1e10(oracle, model, kw, loss):
    w = small_workload(model, 61)
    ref = textbook.per_sample(model, w["graph"], w["x"], w["labels"], w["params"], w["H"], loss=loss, **kw)
    res = _run_oracle(oracle, w, loss=loss, pairing="rowid", precise=True, **kw)
    _compare_tight(res, ref)
    # the reference pairing on a skewed batch: autograd over the round-based dataflow
    tr = oracle.sched_trace(w["graph"])
    ref = textbook.round_based(model, w["graph"], tr, w["x"], w["labels"], w["params"], w["H"],
                               loss=loss, pairing="reference", **kw)
    res = _run_oracle(oracle, w, loss=loss, pairing="reference", precise=True, **kw)
    _compare_tight(res, ref)
    # serial scheduling, weight gradients accumulated per round
    ref = textbook.per_sample(model, w["graph"], w["x"], w["labels"], w["params"], w["H"], loss=loss, **kw)
    res = _run_oracle(oracle, w, loss=loss, batching=False, precise=True, **kw)
    _compare_tight(res, ref)


@pytest.mark.parametrize("model,kw", CASES)
def test_double_build_and_fp32_build_are_the_same_dataflow(oracle, model, kw):
    w = small_workload(model, 62)
    for pairing in ("reference", "rowid"):
        f32 = _run_oracle(oracle, w, pairing=pairing, **kw)
        f64 = _run_oracle(oracle, w, pairing=pairing, precise=True, **kw)
        _compare(f32, f64)


def test_double_build_of_the_ops(oracle):
    r = synth.SplitMix64(63)
    A = r.bulk_uniform(7 * 33, -1, 1).reshape(7, 33)
    B = r.bulk_uniform(33 * 5, -1, 1).reshape(33, 5)
    C0 = r.bulk_uniform(35, -1, 1).reshape(7, 5)
    exact = 0.75 * (A.astype(np.float64) @ B.astype(np.float64)) + 0.5 * C0
    got = oracle.sgemm(0, 0, A, B, alpha=0.75, beta=0.5, Cin=C0, precise=True)
    assert got.dtype == np.float64
    np.testing.assert_allclose(got, exact, rtol=1e-13, atol=1e-14)
    np.testing.assert_allclose(oracle.sgemm(1, 1, A.T.copy(), B.T.copy(), precise=True),
                               A.astype(np.float64) @ B.astype(np.float64), rtol=1e-13, atol=1e-14)
    np.testing.assert_allclose(oracle.colsum(A, precise=True), A.astype(np.float64).sum(0), rtol=1e-14)
    import torch

    logits = r.bulk_uniform(6 * 9, -3, 3).reshape(6, 9)
    labels = np.array([0, 8, 3, 3, 1, 5], np.float32)
    t = torch.tensor(logits, dtype=torch.float64, requires_grad=True)
    rows = torch.nn.functional.cross_entropy(t, torch.tensor(labels, dtype=torch.long), reduction="none")
    rows.mean().backward()
    loss, d = oracle.softmax_xent(logits, labels, precise=True)
    np.testing.assert_allclose(loss, rows.detach().numpy(), rtol=1e-12)
    np.testing.assert_allclose(d, t.grad.numpy(), rtol=1e-11, atol=1e-14)
