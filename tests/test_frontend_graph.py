"""Host-only checks of the front end and the autograd pass: the programs of the three
benchmark applications declare, shape-infer and differentiate (no device needed)."""
import re

import pytest

from cavs_amd import apps


@pytest.fixture
def declare():
    made = []

    def _make(model, **kw):
        a = apps.App(model, opt=-1, **kw)
        made.append(a)
        return a

    yield _make
    for a in made:
        a.close()


def test_tree_lstm_program_and_backward_function(declare):
    a = declare("treelstm", B=2, maxlen=5, V=10, E=3, H=4, C_=5)
    d = a.dump()
    # vertex function: marks of the dynamic edges, graph ops and the four GEMMs of the app
    assert d.count("Gather()") >= 2 and "Scatter(" in d and "Push(" in d and "Pull()" in d
    fwd = d.split("function Node:")[1].split("function Node_grad")[0]
    assert fwd.count("MatMul(") == 4 and fwd.count("Sigmoid(") == 4 and fwd.count("Tanh(") == 2
    assert "[dynamic]" in fwd and re.search(r"Mirror\(Variable_\d+\) -> \(Mirror_\d+\) \[10,3\] ShareMemory=true\n", fwd)
    # GraphOutput received every external edge F reads (weights, sliced biases)
    go = [l for l in d.splitlines() if l.strip().startswith("GraphOutput(")][0]
    assert go.count("Slice_") == 4 and go.count("Reshape_") == 2 and "[-1,4]" in go
    # backward vertex function: Gather <-> Scatter, Pull <-> Push; weight gradients deferred
    per_round = d.split("function Node_grad (per round):")[1].split("function Node_grad (deferred")[0]
    deferred = d.split("function Node_grad (deferred, all rows):")[1].split("backward (main):")[0]
    assert per_round.count("Scatter(") == 2 and "Child=1 Backward=true" in per_round
    assert per_round.count("Gather()") == 1 and per_round.count("Pull()") == 1
    assert per_round.count("MatMul(") == 4        # data gradients stay in the round
    assert deferred.count("MatMul(") == 4         # weight gradients run once over all rows
    assert "EmbeddingLookup_grad" in deferred and "EmbeddingLookup_grad" not in per_round
    assert "MatMul" not in d.split("backward (main):")[1].split("GraphOutput_grad")[0] or True
    main_bwd = d.split("backward (main):")[1]
    assert "SoftmaxEntropyLoss_grad" in main_bwd and "FullyConnected_grad" in main_bwd and "GraphOutput_grad" in main_bwd
    # the sliced biases and weight blocks flow back into their variables
    assert main_bwd.count("PartialAccumulate(") == 6


def test_seq_lstm_and_tree_fc_programs(declare):
    a = declare("lstm", B=3, maxlen=6, V=20, H=4, C_=20)
    d = a.dump()
    fwd = d.split("function Node:")[1].split("function Node_grad")[0]
    assert fwd.count("MatMul(") == 2 and fwd.count("Gather()") == 1
    a.close()
    b = declare("treefc", B=2, maxlen=7, H=4)
    d = b.dump()
    assert "Relu(" in d and "Relu_grad(" in d and "Reduce_sum(" in d
    b.close()
    c = declare("treefc_x", B=2, maxlen=7, H=4)
    d = c.dump()
    assert "Tanh_grad(" in d and "Square(" in d


def test_fusion_pass_groups_the_gate_arithmetic_of_tree_lstm():
    """OPT_FUSION's pass on the Tree-LSTM app, no device needed: the gate arithmetic of F
    becomes one generated kernel, that of the backward function another; the kernel sits
    before the Concat/Scatter that read its results, and broadcast operands wrap."""
    import re
    from cavs_amd import apps

    a = apps.App("treelstm", B=2, maxlen=5, H=8, E=8, V=10, C_=3, opt=-1, lr=0.1)
    try:
        plain, d = a.dump(), a.dump_fused()
    finally:
        a.close()
    assert "FusedKernel" not in plain
    fn = d[d.index("function:"):d.index("function_grad:")]
    bw = d[d.index("function_grad:"):d.index("backward:")]
    assert fn.count("FusedKernel(") == 1 and bw.count("FusedKernel(") == 1
    # every Sigmoid/Tanh/Add/Mul of the gates is inside the kernel, none left as an op
    assert not re.search(r"^  (Sigmoid|Tanh|Mul)\(", fn, re.M)
    assert fn.count("expf(") == 4 and fn.count("tanhf(") == 2
    assert fn.index("FusedKernel(") < fn.index("  Concat(") < fn.index("  Scatter(")
    # the kernel keeps the reference's signature: outputs, const inputs, counts, n_elements
    sig = re.search(r'extern "C" __global__ void (FusedKernel_\d+)\((.*?)\)\n', fn, re.S).group(2)
    kinds = [("out" if p.startswith("float *") else "in" if p.startswith("const float *") else "count")
             for p in sig.split(", ")]
    assert kinds[-1] == "count" and sig.endswith("const int n_elements")
    assert kinds == sorted(kinds, key=["out", "in", "count"].index)
    assert kinds.count("count") == kinds.count("out") + kinds.count("in") + 1
    # a bias row is a broadcast operand; a per-vertex slab is indexed directly
    assert re.search(r"tmp_Mirror_\d+ = Mirror_\d+\[idx % Mirror_\d+_count\]", fn)
    assert re.search(r"tmp_Slice_\d+ = Slice_\d+\[idx\]", fn)
    # the backward kernel accumulates onto gradients that an earlier op already wrote
    assert re.search(r"float tmp_(\w+_grad) = \1\[idx\] \+ \(", bw)


def test_fusion_pass_keeps_small_groups_unfused():
    """A group pays only with two or more arithmetic members (cavs/midend/runtime_compiler/parser.cc:118-131)."""
    from cavs_amd import apps

    a = apps.App("treefc", B=2, maxlen=5, H=8, opt=-1, lr=0.1)
    try:
        d = a.dump_fused()
    finally:
        a.close()
    fn = d[d.index("function:"):d.index("function_grad:")]
    assert "FusedKernel(" not in fn  # forward F has a single Relu


def test_fusion_pass_takes_bias_gradients_in_as_reducing_outputs():
    """The gradient of a bias is a sum over the rows of a per-row value.  The pass takes those
    deferred ops into the per-round backward kernel as outputs narrower than the element range,
    stored with atomicAdd onto out[idx % out_count] (cavs/midend/runtime_compiler/
    code_generator.cc:84-100) and listed in ZeroEnforced; what reads the sums stays deferred."""
    import re
    from cavs_amd import apps

    for model, reduced in (("treefc_x", 1), ("treelstm", 5), ("lstm", 4)):
        a = apps.App(model, B=2, maxlen=7, H=8, E=8, V=10, C_=3, opt=-1, lr=0.1)
        try:
            d = a.dump_fused()
        finally:
            a.close()
        bw = d[d.index("function_grad:"):d.index("function_grad_deferred:")]
        deferred = d[d.index("function_grad_deferred:"):d.index("backward:")]
        stores = re.findall(r"atomicAdd\(&(\w+)\[idx % \1_count\], tmp_\1\);", bw)
        assert len(stores) == reduced, (model, stores)
        for name in stores:
            assert f"{name}[idx] =" not in bw                       # never stored as a full-range output
            assert not re.search(rf"= {name}\[idx", bw)             # nor read back
            assert re.search(rf"^  \w+\({name}[,)]", deferred, re.M)  # its reader runs after the loop
            assert not re.search(rf"-> \({name}\)", deferred)       # the op that produced it is gone from there
