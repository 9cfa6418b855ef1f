"""The C++ front end (Sym / GraphSupport / Session), its autograd pass and the op-by-op
execution of F on the GPU, against the oracle on the same seeded inputs."""
import numpy as np
import pytest

from cavs_amd import apps, session, synth
from test_oracle_models import small_workload
from tolerance import close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"


def oracle_step(oracle, w, model, **kw):
    # the oracle's dataflow in double: what the fp32 results are held to 1e-4 relative / 1e-5 absolute against
    return oracle.model_step(model, w["graph"], w["x"], w["labels"], w["params"], H=w["H"], E=w["E"], V=w["V"],
                             Cc=w["C"], precise=True, threads=16, **kw)


def run_app(model, w, *, opt, pairing, allow_fused, root_mask=None, want_generated=False):
    B, maxlen = w["graph"].shape
    a = apps.App(model, B=B, maxlen=maxlen, H=w["H"], E=w["E"], V=w["V"], C_=w["C"], opt=opt, lr=0.0,
                 pairing=pairing, allow_fused=allow_fused)
    names = {"treelstm": ("Emb", "W", "U", "Bv", "Wfc", "bfc"), "lstm": ("Emb", "W", "Bv", "Wfc", "bfc"),
             "treefc": ("W",), "treefc_x": ("W", "Bv")}[model]
    a.set_params({k: w["params"][k] for k in names})
    print(f"[case] app={model} N={w['N']} opt={opt} pairing={pairing} fused_allowed={allow_fused}", flush=True)
    loss, go = a.step(w["graph"], w["x"], w["labels"], train=True, root_mask=root_mask)
    H, E, V, C = w["H"], w["E"], w["V"], w["C"]
    shapes = {"Emb": (V, E), "W": {"treelstm": (E, 4 * H), "lstm": (8 * H * H,), "treefc": (2 * H, H), "treefc_x": (2 * H, H)}[model],
              "U": (4 * H * H,), "Bv": (H,) if model.startswith("treefc") else (4 * H,), "Wfc": (C, H), "bfc": (C,)}
    grads = {"d" + k: a.grad(k, shapes[k]) for k in names}
    fused = a.fused
    generated = a.generated_kernels
    a.close()
    if want_generated:
        return loss, go, grads, fused, generated
    return loss, go, grads, fused


@pytest.mark.parametrize("model", ["treelstm", "lstm"])
@pytest.mark.parametrize("pairing", ["reference", "rowid"])
@pytest.mark.parametrize("opt", [session.OPT_BATCHING, 0])
def test_op_by_op_path_matches_oracle(oracle, model, pairing, opt):
    w = small_workload(model, 81, B=5, H=8, E=6, V=23, C=4)
    want = oracle_step(oracle, w, model, pairing=pairing, batching=bool(opt))
    loss, go, grads, fused = run_app(model, w, opt=opt, pairing=pairing, allow_fused=False)
    assert not fused
    close(go, want["graph_out"], "graph_out")
    close(loss, want["loss"], "loss")
    for k, v in grads.items():
        close(v, want["grads"][k], k)


@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_tree_fc_apps_op_by_op(oracle, pairing):
    w = small_workload("treefc", 82, B=5, H=8)
    # the reference app: relu, no bias, no input, loss = Reduce_sum (sum of |h|, gradient 1)
    want = oracle_step(oracle, w, "treefc", pairing=pairing, loss="sum_abs", act=0)
    loss, go, grads, _ = run_app("treefc", w, opt=session.OPT_BATCHING, pairing=pairing, allow_fused=False)
    close(go, want["graph_out"], "graph_out")
    close(loss, want["loss"], "loss")
    close(grads["dW"], want["grads"]["dW"], "dW")
    # tanh + bias + Pull'ed input, sum of squares at the roots through Square * mask
    want = oracle_step(oracle, w, "treefc", pairing=pairing, loss="root_sq", act=1, use_bias=True, use_x=True)
    N, H = w["N"], w["H"]
    mask = np.zeros((N, H), np.float32)
    off = 0
    for row in w["graph"]:
        n = int(np.argmax(row == -1)) + 1
        mask[off + n - 1] = 1
        off += n
    loss, go, grads, _ = run_app("treefc_x", w, opt=session.OPT_BATCHING, pairing=pairing, allow_fused=False, root_mask=mask)
    close(go, want["graph_out"], "graph_out")
    close(loss, want["loss"], "loss")
    close(grads["dW"], want["grads"]["dW"], "dW")
    close(grads["dBv"], want["grads"]["dBv"], "dBv")


@pytest.mark.parametrize("model", ["treelstm", "lstm", "treefc", "treefc_x"])
@pytest.mark.parametrize("pairing", ["reference", "rowid"])
def test_recognised_vertex_functions_run_on_the_fused_round_kernels(oracle, model, pairing):
    """Session(OPT_BATCHING) on the benchmark apps: F is recognised and lowered onto the
    fused kernels; results must equal the oracle (and hence the op-by-op path)."""
    base = {"treefc_x": "treefc"}.get(model, model)
    w = small_workload(base, 83, B=6, H=16, E=12, V=29, C=5)
    mask, kw = None, {}
    if model == "treefc":
        kw = dict(loss="sum_abs", act=0)
    elif model == "treefc_x":
        kw = dict(loss="root_sq", act=1, use_bias=True, use_x=True)
        mask = np.zeros((w["N"], w["H"]), np.float32)
        off = 0
        for row in w["graph"]:
            n = int(np.argmax(row == -1)) + 1
            mask[off + n - 1] = 1
            off += n
    want = oracle_step(oracle, w, base, pairing=pairing, **kw)
    loss, go, grads, fused = run_app(model, w, opt=session.OPT_BATCHING, pairing=pairing, allow_fused=True, root_mask=mask)
    assert fused, "the vertex function was not recognised"
    close(go, want["graph_out"], "graph_out")
    close(loss, want["loss"], "loss")
    for k, v in grads.items():
        close(v, want["grads"][k], k)


def test_serial_sessions_are_never_lowered(oracle):
    w = small_workload("lstm", 84, B=3, H=8)
    _, _, _, fused = run_app("lstm", w, opt=0, pairing="reference", allow_fused=True)
    assert not fused


def test_training_steps_update_variables_like_the_oracle(oracle):
    """Three SGD steps through Session::Run({train}) on the fused path."""
    w = small_workload("treelstm", 85, B=4, H=8, E=6, V=19, C=3)
    B, maxlen = w["graph"].shape
    lr = 0.5
    a = apps.App("treelstm", B=B, maxlen=maxlen, H=8, E=6, V=19, C_=3, opt=session.OPT_BATCHING, lr=lr)
    a.set_params(w["params"])
    p = {k: np.array(v, np.float32) for k, v in w["params"].items()}
    for step in range(3):
        print(f"[case] sgd step {step}", flush=True)
        want = oracle_step(oracle, dict(w, params=p), "treelstm")
        loss, _ = a.step(w["graph"], w["x"], w["labels"], train=True)
        close(loss, want["loss"], f"loss at step {step}")
        for k in ("Emb", "W", "U", "Bv", "Wfc", "bfc"):
            p[k] = (p[k] - np.float32(lr) * want["grads"]["d" + k].reshape(p[k].shape)).astype(np.float32)
    close(a.grad("W", (6, 32), grad=False), p["W"], "W after 3 steps")
    a.close()


@pytest.mark.parametrize("model,H", [("treelstm", 128), ("lstm", 256)])
def test_training_steps_at_sizes_whose_rounds_read_packed_weights(oracle, model, H):
    """Rounds of 70 vertices at these hidden sizes read the recurrent weights from a tile-major
    copy.  The parameters live in the Variables' own tensors and the optimizer is an ordinary op
    of the main scope: the first forward pass packs on demand, later ones read the copy that the
    optimizer's update of that Variable keeps current.  Losses and the final weights against the
    oracle over three steps."""
    E, V, C_ = (16 if model == "treelstm" else H), 37, 5
    w = small_workload(model, 334, B=70, H=H, E=E, V=V, C=C_, skew=False)
    rec = "U" if model == "treelstm" else "W"
    names = ("Emb", "W", "U", "Bv", "Wfc", "bfc") if model == "treelstm" else ("Emb", "W", "Bv", "Wfc", "bfc")
    p = {k: np.array(w["params"][k], np.float32) for k in names}
    p[rec] = (p[rec] * np.float32(0.2)).astype(np.float32)
    B, maxlen = w["graph"].shape
    lr = 0.25
    a = apps.App(model, B=B, maxlen=maxlen, H=H, E=E, V=V, C_=C_, opt=session.OPT_BATCHING, lr=lr)
    a.set_params(p)
    for step in range(3):
        print(f"[case] front end, packed weights, {model} step {step}", flush=True)
        want = oracle_step(oracle, dict(w, params=p), model)
        loss, _ = a.step(w["graph"], w["x"], w["labels"], train=True)
        close(loss, want["loss"], f"loss at step {step}")
        for k in names:
            p[k] = (p[k] - np.float32(lr) * want["grads"]["d" + k].reshape(p[k].shape)).astype(np.float32)
    close(a.grad(rec, p[rec].shape, grad=False), p[rec], f"{rec} after 3 steps")
    a.close()


def _root_mask(w):
    mask = np.zeros((w["N"], w["H"]), np.float32)
    off = 0
    for row in w["graph"]:
        n = int(np.argmax(row == -1)) + 1
        mask[off + n - 1] = 1
        off += n
    return mask


@pytest.mark.parametrize("model", ["treelstm", "lstm", "treefc", "treefc_x"])
@pytest.mark.parametrize("opt", [session.OPT_BATCHING | session.OPT_FUSION, session.OPT_FUSION])
def test_generated_kernels_of_the_fusion_pass_match_oracle(oracle, model, opt):
    """OPT_FUSION on the op-by-op path: the elementwise groups of F and of its backward
    function run as kernels generated and compiled at run time; values must not move."""
    base = {"treefc_x": "treefc"}.get(model, model)
    w = small_workload(base, 86, B=5, H=8, E=6, V=23, C=4)
    mask, kw = None, {}
    if model == "treefc":
        kw = dict(loss="sum_abs", act=0)
    elif model == "treefc_x":
        kw = dict(loss="root_sq", act=1, use_bias=True, use_x=True)
        mask = _root_mask(w)
    want = oracle_step(oracle, w, base, batching=bool(opt & session.OPT_BATCHING), **kw)
    loss, go, grads, fused, generated = run_app(model, w, opt=opt, pairing="reference", allow_fused=False,
                                                root_mask=mask, want_generated=True)
    assert not fused
    assert generated >= 1
    close(go, want["graph_out"], "graph_out")
    close(loss, want["loss"], "loss")
    for k, v in grads.items():
        close(v, want["grads"][k], k)


def test_reference_smoke_programs_print_their_known_values():
    """session_test.cc and fusion_session_test.cc of the reference, same programs, same feeds."""
    import ctypes as C
    import json
    import os

    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "smoke_kats.json")))
    lib, _ = apps.libs()
    out = (C.c_float * 6)()
    assert lib.cavs_smoke_session_add(out) == 0
    np.testing.assert_array_equal(np.array(out[:]), np.array(kat["session_add"]["expect"], np.float32))
    for opt, expect_kernels in ((session.OPT_FUSION, 2), (0, 0)):
        e, yy, n = (C.c_float * 6)(), (C.c_float * 4)(), C.c_int(-1)
        assert lib.cavs_smoke_fusion(opt, e, yy, C.byref(n)) == 0
        np.testing.assert_allclose(np.array(e[:]), np.array(kat["fusion_E"]["expect"], np.float32), rtol=1e-6)
        np.testing.assert_allclose(np.array(yy[:]), np.array(kat["fusion_YY"]["expect"], np.float32), rtol=1e-6)
        assert n.value == expect_kernels


def test_optimizer_with_gradient_clipping(oracle):
    """Optimizer(vars, lr, clip): gradients are scaled by clip / max(sum of norms, clip) before
    w -= lr * g (cavs/backend/op_impl_clip.cu); the threshold is chosen below the sum of norms."""
    w = small_workload("treelstm", 87, B=4, H=8, E=6, V=19, C=3)
    B, maxlen = w["graph"].shape
    names = ("Emb", "W", "U", "Bv", "Wfc", "bfc")
    want = oracle_step(oracle, w, "treelstm")
    norms = sum(float(np.sqrt((want["grads"]["d" + k].astype(np.float64) ** 2).sum())) for k in names)
    clip, lr = 0.25 * norms, 0.5
    a = apps.App("treelstm", B=B, maxlen=maxlen, H=8, E=6, V=19, C_=3, opt=session.OPT_BATCHING, lr=lr, clip=clip)
    a.set_params(w["params"])
    a.step(w["graph"], w["x"], w["labels"], train=True)
    shapes = {"Emb": (19, 6), "W": (6, 32), "U": (4 * 64,), "Bv": (32,), "Wfc": (3, 8), "bfc": (3,)}
    for k in names:
        p0 = np.asarray(w["params"][k], np.float32).reshape(shapes[k])
        step = np.float32(lr) * np.float32(0.25) * want["grads"]["d" + k].reshape(shapes[k])
        close(a.grad(k, shapes[k], grad=False), p0 - step, f"{k} after a clipped step")
    a.close()


@pytest.mark.parametrize("allow_fused", [True, False])
def test_optimizer_iters_runs_the_training_scope_that_many_times_per_run(allow_fused):
    """Optimizer(vars, lr, clip, iters): one Session::Run makes `iters` passes of forward, backward
    and update (ScopedNode(s_, name, iters), cavs/midend/graph_util.cc:266-283).  One Run with
    iters=3 leaves the variables where three Runs with iters=1 leave them (up to the summation order
    of the embedding gradient's atomics)."""
    w = small_workload("lstm", 88, B=4, H=16, V=19, C=4)
    B, maxlen = w["graph"].shape
    finals = []
    for iters, runs in ((1, 3), (3, 1)):
        a = apps.App("lstm", B=B, maxlen=maxlen, H=16, E=16, V=19, C_=4, opt=session.OPT_BATCHING, lr=0.25, iters=iters,
                     allow_fused=allow_fused)
        a.set_params(w["params"])
        for _ in range(runs):
            print(f"[case] iters={iters} fused={allow_fused}", flush=True)
            a.step(w["graph"], w["x"], w["labels"], train=True)
        finals.append({k: a.grad(k, shp, grad=False) for k, shp in (("W", (8 * 16 * 16,)), ("Bv", (64,)), ("Wfc", (4, 16)))})
        a.close()
    assert not np.array_equal(finals[0]["W"], np.asarray(w["params"]["W"], np.float32).ravel())
    for k in finals[0]:
        close(finals[0][k], finals[1][k], k, rtol=1e-5, atol=1e-6)
