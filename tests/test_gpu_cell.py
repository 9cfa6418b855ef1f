"""Vertex functions lowered onto kernels generated for them: the reference's three applications
forced onto that path, a Tree-LSTM with a forget-gate matrix per child, a gated cell with one state
block and a tree GRU (two stages of products: a chain of two cells), against the oracle (or, where
the oracle has no restatement, the fp64 autograd formulation of tests/textbook.py) on the same
seeded inputs."""
import numpy as np
import pytest

import textbook
from cavs_amd import apps, session, synth
from test_cell_lowering import CELL_SEEDS, CHAIN_SEEDS
from test_oracle_models import small_workload
from tolerance import close

pytestmark = pytest.mark.gpu

NAMES = {"treelstm": ("Emb", "W", "U", "Bv", "Wfc", "bfc"), "treelstm2": ("Emb", "W", "U", "Bv", "Wfc", "bfc"),
         "treegate": ("Emb", "W", "U", "Bv", "Wfc", "bfc"), "treegru": ("Emb", "W", "U", "Bv", "Wfc", "bfc"), "treedeep": ("Emb", "W", "U", "Bv", "Wfc", "bfc"), "lstm": ("Emb", "W", "Bv", "Wfc", "bfc"), "treefc": ("W",), "treefc_x": ("W", "Bv")}


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"


def oracle_step(oracle, w, model, **kw):
    return oracle.model_step(model, w["graph"], w["x"], w["labels"], w["params"], H=w["H"], E=w["E"], V=w["V"],
                             Cc=w["C"], precise=True, threads=16, **kw)


def run_generated(model, w, pairing, mode=2, lr=0.0, root_mask=None):
    B, maxlen = w["graph"].shape
    a = apps.App(model, B=B, maxlen=maxlen, H=w["H"], E=w["E"], V=w["V"], C_=w["C"], opt=session.OPT_BATCHING, lr=lr,
                 pairing=pairing, allow_fused=mode)
    a.set_params({k: w["params"][k] for k in NAMES[model]})
    print(f"[case] app={model} N={w['N']} H={w['H']} pairing={pairing} lowering mode={mode}", flush=True)
    loss, go = a.step(w["graph"], w["x"], w["labels"], train=True, root_mask=root_mask)
    grads = {"d" + k: a.grad(k, np.shape(w["params"][k])) for k in NAMES[model]}
    kind = a.fused_kind
    a.close()
    return loss, go, grads, kind


def compare(got, want):
    loss, go, grads, _ = got
    close(go, want["graph_out"], "graph_out")
    close(loss, want["loss"], "loss")
    for k, v in grads.items():
        close(v, np.reshape(want["grads"][k], v.shape), k)


@pytest.mark.parametrize("model,H", [("treelstm", 32), ("treelstm", 64), ("treelstm", 128), ("treelstm", 256), ("lstm", 64), ("treefc", 32), ("treefc", 128)])
@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_the_reference_applications_on_generated_kernels(oracle, model, H, pairing):
    """Lowering mode 2 skips the hand-written kernels: the same F, recognised by its shape alone.
    Mode 3 also runs the backward rounds as a batch whose message flow is no forest needs them: two
    launches per round, with the message gradients going through the gradient of the message pool."""
    w = small_workload(model, 183, B=6, H=H, E=12, V=29, C=5)
    kw = dict(loss="sum_abs", act=0) if model == "treefc" else {}
    want = oracle_step(oracle, w, model, pairing=pairing, **kw)
    for mode in (2, 3):
        got = run_generated(model, w, pairing, mode=mode)
        assert got[3] == 2, "the vertex function was not lowered onto generated kernels"
        compare(got, want)


@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_a_pulled_row_of_the_vertex_input_on_generated_kernels(oracle, pairing):
    """Tree-FC with tanh, a bias and the vertex's own input row added in: the row is read by vertex id
    inside the round kernels (Pull folded in), the loss is the sum of squares at the roots."""
    w = small_workload("treefc", 188, B=6, H=64)
    want = oracle_step(oracle, w, "treefc", pairing=pairing, loss="root_sq", act=1, use_bias=True, use_x=True)
    mask = np.zeros((w["N"], w["H"]), np.float32)
    off = 0
    for row in w["graph"]:
        n = int(np.argmax(row == -1)) + 1
        mask[off + n - 1] = 1
        off += n
    for mode in (2, 3):
        got = run_generated("treefc_x", w, pairing, mode=mode, root_mask=mask)
        assert got[3] == 2
        compare(got, want)


@pytest.mark.parametrize("H", [64, 128])
@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_a_tree_lstm_with_a_forget_matrix_per_child(oracle, H, pairing):
    """A fourth vertex function, which no hand-written kernel covers: lowered by the default mode."""
    w = small_workload("treelstm2", 184, B=7, H=H, E=20, V=31, C=4)
    want = oracle_step(oracle, w, "treelstm2", pairing=pairing)
    got = run_generated("treelstm2", w, pairing, mode=1)
    assert got[3] == 2
    compare(got, want)
    # and op by op, the way the reference would run it
    compare(run_generated("treelstm2", w, pairing, mode=0), want)


def test_a_gated_cell_with_one_state_block_against_fp64_autograd():
    """Children's states enter through products (one of them over their concatenation) and
    elementwise; the message has one block.  No oracle restatement: held to the per-sample fp64
    formulation, which a batch under row-id pairing equals."""
    w = small_workload("treegate", 185, B=6, H=64, E=12, V=29, C=5)
    want = textbook.per_sample("treegate", w["graph"], w["x"], w["labels"], w["params"], w["H"])
    for mode in (1, 3):
        got = run_generated("treegate", w, "rowid", mode=mode)
        assert got[3] == 2
        compare(got, want)
    compare(run_generated("treegate", w, "rowid", mode=0), want)


@pytest.mark.parametrize("H", [32, 64, 128])
def test_a_tree_gru_runs_as_a_chain_of_two_cells_against_fp64_autograd(H):
    """The candidate's product takes r * (h_l + h_r) as its left operand, which depends on the
    products behind r: two launches per round and direction (four backward when the message flow
    is no forest, which mode 3 forces).  Held to the per-sample fp64
    formulation under row-id pairing, and to the same program run operator by operator under the
    reference's pairing."""
    w = small_workload("treegru", 186, B=6, H=H, E=12, V=29, C=5)
    want = textbook.per_sample("treegru", w["graph"], w["x"], w["labels"], w["params"], w["H"])
    for mode in (1, 3):
        got = run_generated("treegru", w, "rowid", mode=mode)
        assert got[3] == 2
        compare(got, want)
    by_op = run_generated("treegru", w, "rowid", mode=0)
    compare(by_op, want)
    ref_pairing = run_generated("treegru", w, "reference", mode=0)
    got = run_generated("treegru", w, "reference", mode=1)
    assert got[3] == 2
    compare(got, dict(loss=ref_pairing[0], graph_out=ref_pairing[1], grads=ref_pairing[2]))


@pytest.mark.parametrize("H", [32, 128])
def test_three_stages_that_share_a_weight_block_a_block_of_xw_and_a_bias(H):
    """A chain of three cells whose weight gradients meet: the first and the third cell multiply by
    the same block (the second's share is added one launch later), read the same block of x W
    (likewise for d W and d e), and the first two add the same bias."""
    w = small_workload("treedeep", 189, B=6, H=H, E=12, V=29, C=5)
    want = textbook.per_sample("treedeep", w["graph"], w["x"], w["labels"], w["params"], w["H"])
    for mode in (1, 3):
        got = run_generated("treedeep", w, "rowid", mode=mode)
        assert got[3] == 2
        compare(got, want)
    compare(run_generated("treedeep", w, "rowid", mode=0), want)


@pytest.mark.parametrize("seed", CELL_SEEDS + CHAIN_SEEDS)
def test_a_family_of_cells_lowered_and_op_by_op(seed):
    """cell<seed>: one or two children, one or two state blocks, three or four gates over the first
    child, the last child, the children's sum or their concatenation, sigmoid or tanh each; for
    the chain seeds one or two of the gates over another gate times those (two or three stages of
    products).  No restatement of these exists anywhere else: the generated kernels are held to
    the same program run operator by operator (each operator of which the oracle pins), and the
    two backward forms to each other."""
    two = seed & 1
    H, E, V, C_ = 64, 12, 29, 5
    w = small_workload("treelstm" if two else "lstm", 190 + seed % 7, B=6, H=H, E=E, V=V, C=C_)
    w = dict(w, E=E)  # (the chain workload sets E = H for its own model)
    B, maxlen = w["graph"].shape
    rng = synth.SplitMix64(seed)
    res = {}
    for mode in (1, 3, 0):
        a = apps.App(f"cell{seed}", B=B, maxlen=maxlen, H=H, E=E, V=V, C_=C_, opt=session.OPT_BATCHING, lr=0.0, pairing="rowid",
                     allow_fused=mode)
        if mode == 1:
            sizes = {k: a.var_size(k) for k in ("Emb", "W", "U", "Bv")}
            # (a chain's stages multiply one after the other: with +-0.4 at H = 64 the gain per stage is
            # about 3 and the two paths' fp32 summation orders show, up to 5e-4 relative in single
            # entries of one seed's gradients; with +-0.2 every tensor stays within 2 % of the tolerance)
            amp = 0.2 if seed >> 16 else 0.4
            p = {k: rng.bulk_uniform(n, -amp, amp) for k, n in sizes.items()}
            p["Wfc"], p["bfc"] = w["params"]["Wfc"], w["params"]["bfc"]
        a.set_params(p)
        print(f"[case] cell{seed} children={1 + two} N={w['N']} lowering mode={mode}", flush=True)
        loss, go = a.step(w["graph"], w["x"], w["labels"], train=True)
        assert a.fused_kind == (2 if mode else 0)
        res[mode] = dict(loss=loss, graph_out=go, grads={"d" + k: a.grad(k, (np.size(v),)) for k, v in p.items()})
        a.close()
    for mode in (1, 3):
        compare((res[mode]["loss"], res[mode]["graph_out"], res[mode]["grads"], 2), res[0])


def test_training_steps_on_generated_kernels_update_variables_like_the_oracle(oracle):
    """Three SGD steps of the fourth vertex function through Session::Run({train})."""
    H, E, V, C_ = 64, 10, 23, 4
    w = small_workload("treelstm2", 187, B=5, H=H, E=E, V=V, C=C_)
    B, maxlen = w["graph"].shape
    lr = 0.25
    a = apps.App("treelstm2", B=B, maxlen=maxlen, H=H, E=E, V=V, C_=C_, opt=session.OPT_BATCHING, lr=lr)
    p = {k: np.array(w["params"][k], np.float32) for k in NAMES["treelstm2"]}
    p["U"] = (p["U"] * np.float32(0.3)).astype(np.float32)
    a.set_params(p)
    for step in range(3):
        print(f"[case] generated kernels, sgd step {step}", flush=True)
        want = oracle_step(oracle, dict(w, params=p), "treelstm2")
        loss, _ = a.step(w["graph"], w["x"], w["labels"], train=True)
        assert a.fused_kind == 2
        close(loss, want["loss"], f"loss at step {step}")
        for k in NAMES["treelstm2"]:
            p[k] = (p[k] - np.float32(lr) * want["grads"]["d" + k].reshape(p[k].shape)).astype(np.float32)
    close(a.grad("U", p["U"].shape, grad=False), p["U"], "U after 3 steps")
    close(a.grad("Bv", p["Bv"].shape, grad=False), p["Bv"], "Bv after 3 steps")
    a.close()


@pytest.mark.parametrize("model", ["treegru", "treedeep"])
def test_training_steps_of_a_chain_of_cells_over_changing_batches(model):
    """Three SGD steps, each on another batch (other trees, other words): what a step leaves behind
    -- the rows of the embedding gradient it touched, bias and weight gradients that several cells
    add their shares to -- must not show in the next one.  Held to fp64 autograd step by step."""
    H, E, V, C_ = 64, 10, 23, 4
    lr = 0.2
    batches = [small_workload(model, 300 + i, B=5, H=H, E=E, V=V, C=C_) for i in range(3)]
    B = max(b["graph"].shape[0] for b in batches)
    maxlen = max(b["graph"].shape[1] for b in batches)
    a = apps.App(model, B=B, maxlen=maxlen, H=H, E=E, V=V, C_=C_, opt=session.OPT_BATCHING, lr=lr, pairing="rowid")
    p = {k: np.array(batches[0]["params"][k], np.float64) for k in NAMES[model]}
    a.set_params({k: v.astype(np.float32) for k, v in p.items()})
    for step, w in enumerate(batches):
        assert w["graph"].shape == (B, maxlen)
        print(f"[case] {model} on a chain of cells, sgd step {step}, N={w['N']}", flush=True)
        want = textbook.per_sample(model, w["graph"], w["x"], w["labels"], {k: v.astype(np.float32) for k, v in p.items()}, H)
        loss, _ = a.step(w["graph"], w["x"], w["labels"], train=True)
        assert a.fused_kind == 2
        close(loss, want["loss"], f"loss at step {step}")
        for k in NAMES[model]:
            p[k] = p[k] - lr * want["grads"]["d" + k].reshape(p[k].shape)
    for k in NAMES[model]:
        close(a.grad(k, p[k].shape, grad=False), p[k], f"{k} after 3 steps")
    a.close()
