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
