"""The C++ front end (Sym / GraphSupport / Session), its autograd pass and the op-by-op
execution of F on the GPU, against the oracle on the same seeded inputs."""
import numpy as np
import pytest

from cavs_amd import apps, session, synth
from test_gpu_models import close
from test_oracle_models import small_workload

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"


def oracle_step(oracle, w, model, **kw):
    return oracle.model_step(model, w["graph"], w["x"], w["labels"], w["params"], H=w["H"], E=w["E"], V=w["V"],
                             Cc=w["C"], **kw)


def run_app(model, w, *, opt, pairing, allow_fused, root_mask=None):
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
    a.close()
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
